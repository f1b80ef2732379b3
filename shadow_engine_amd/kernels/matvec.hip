// Matrix-vector products over GGUF row-major quantized matrices (Q8_0, IQ3_S) for 1..4 inputs at a time.
//
// Shape of every fast kernel here: a workgroup of 256 threads (4 waves of 64) owns `rpb` consecutive rows.  The rows'
// bytes are one contiguous span of the matrix, so the workgroup streams them from HBM with 16-byte loads, lane after
// lane, into LDS; nothing about the 34-byte (Q8_0) or 110-byte (IQ3_S) block boundaries matters to the HBM side.  Each
// lane then decodes one unit of 32 weights from LDS against inputs it holds in registers, and a segment of lanes is
// summed with wave shuffles.  Follows the semantics of the reference's matvec_cols_* / matvec_grouped_* kernels
// (kernels/matvec.cu:677-756, 1576-1677): y_j = W x_j with the weights decoded once for all inputs.

struct Q80 {
    static constexpr u32 QK = 32, BB = 34;
};
struct IQ3S {
    static constexpr u32 QK = 256, BB = 110;
};

// ------------------------------------------------------------------------------------------------ reference kernels
// One wave a row, a lane every 64th weight, each weight decoded on its own from global memory: correct for any column
// count that is a whole number of blocks; the kernel GpuBackend::matvec uses (crates/shadowzero-cuda/src/backend.rs:57-101, matvec.cu:7-32).
__device__ __forceinline__ float q8_0_at(const u8* row, u32 i) {
    const u8* b = row + (u64) (i / 32) * 34;
    const float d = f16_to_f32((u16) (b[0] | (b[1] << 8)));
    return d * (float) (i8) b[2 + (i % 32)];
}

__device__ __forceinline__ float iq3_s_at(const u8* row, u32 i) {
    const u8* b = row + (u64) (i / 256) * 110;
    const u32 e = i % 256, j = e / 4, g = e / 32;
    const float d = f16_to_f32((u16) (b[0] | (b[1] << 8)));
    const u32 idx = b[2 + j] | (((b[66 + j / 8] >> (j % 8)) & 1u) << 8);
    const u32 s = (b[106 + g / 2] >> (4 * (g % 2))) & 0x0f;
    const float db = d * (float) (1 + 2 * s);
    const float grid = (float) ((IQ3S_GRID[idx] >> (8 * (e % 4))) & 0xff);
    const float sg = ((b[74 + e / 8] >> (e % 8)) & 1) ? -1.0f : 1.0f;
    return db * grid * sg;
}

extern "C" __global__ void __launch_bounds__(256) matvec_q8_0(const u8* w, const float* x, float* y, u32 rows, u32 cols) {
    const u32 r = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    if (r >= rows) return;
    const u8* row = w + (u64) r * (cols / 32 * 34);
    float acc = 0.0f;
    for (u32 i = lane; i < cols; i += 64) acc = __builtin_fmaf(q8_0_at(row, i), x[i], acc);
    acc = seg_sum<64>(acc, lane);
    if (lane == 0) y[r] = acc;
}

extern "C" __global__ void __launch_bounds__(256) matvec_iq3_s(const u8* w, const float* x, float* y, u32 rows, u32 cols) {
    const u32 r = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    if (r >= rows) return;
    const u8* row = w + (u64) r * (cols / 256 * 110);
    float acc = 0.0f;
    for (u32 i = lane; i < cols; i += 64) acc = __builtin_fmaf(iq3_s_at(row, i), x[i], acc);
    acc = seg_sum<64>(acc, lane);
    if (lane == 0) y[r] = acc;
}

// Whole blocks to f32, a thread a weight, in the CPU reference's operation order (quant.rs:148-179): bit-exact test hooks.
extern "C" __global__ void __launch_bounds__(256) dequant_q8_0(const u8* w, float* out, u64 n) {
    const u64 i = (u64) blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = q8_0_at(w + (i / 32) * 34, (u32) (i % 32));
}

extern "C" __global__ void __launch_bounds__(256) dequant_iq3_s(const u8* w, float* out, u64 n) {
    const u64 i = (u64) blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = iq3_s_at(w + (i / 256) * 110, (u32) (i % 256));
}

// ------------------------------------------------------------------------------------------------------ LDS staging
extern __shared__ u32 sz_dyn_lds[];

// Copies bytes [g0, g0 + span) of global memory to LDS so that byte g0 lands at LDS byte (g0 & 15): whole 16-byte
// chunks, one per thread per step, except a first or last chunk that would reach outside the span, which is read
// byte by byte so that the kernel never touches memory outside the matrix.
__device__ __forceinline__ u32 stage_span(const u8* g0, u32 span, u32 tid) {
    const u32 head = (u32) ((u64) g0 & 15);
    const u8* a0 = g0 - head;
    const u32 total = head + span;
    const u32 nchunks = (total + 15) / 16;
    if (head == 0 && total % 16 == 0) {
        // the usual case, whole chunks only: four a thread a round, their loads all in flight before the first store (a
        // load-store loop takes a memory round trip a chunk); a thread past the end reads the last chunk again and drops it
        for (u32 c0 = 0; c0 < nchunks; c0 += 1024) {
            u32x4 v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = *(const u32x4*) (a0 + (u64) min(c0 + tid + 256 * i, nchunks - 1) * 16);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 c = c0 + tid + 256 * i;
                if (c < nchunks) ((u32x4*) sz_dyn_lds)[c] = v[i];
            }
        }
        return head;
    }
    for (u32 c = tid; c < nchunks; c += 256) {
        u32x4 v;
        if ((c == 0 && head != 0) || (c * 16 + 16 > total)) {
            u32 w[4] = {0, 0, 0, 0};
            for (u32 b = 0; b < 16; b++) {
                const u32 idx = c * 16 + b;
                if (idx >= head && idx < total) w[b / 4] |= (u32) a0[idx] << (8 * (b % 4));
            }
            v = u32x4{w[0], w[1], w[2], w[3]};
        } else {
            v = *(const u32x4*) (a0 + c * 16);
        }
        ((u32x4*) sz_dyn_lds)[c] = v;
    }
    return head;
}

__device__ __forceinline__ u32 lds_u8(u32 o) { return ((const u8*) sz_dyn_lds)[o]; }
__device__ __forceinline__ u32 lds_u16(u32 o) { return ((const u16*) sz_dyn_lds)[o >> 1]; }   // o even
__device__ __forceinline__ u32 lds_u32(u32 o) { return sz_dyn_lds[o >> 2]; }                  // o multiple of 4

// ------------------------------------------------------------------------------------------------------- unit dots
// out[j] = sum over the unit's 32 weights of w_i * x[i][j], the block scale included.  `o` is the LDS byte offset of the
// unit's row; `u` the unit's index in the row.
template <int M>
__device__ __forceinline__ void unit_dot_q8_0(u32 o, u32 u, const float (&x)[32][M], float (&out)[M]) {
    const u32 b = o + 34 * u;
    const float d = f16_to_f32((u16) lds_u16(b));
    const u32 q0 = b + 2;                       // the 32 codes; q0 is 0 or 2 modulo 4
    const u32 sh = (q0 & 3) * 8;
    const u32 a = q0 & ~3u;
    u32 dw[9];
#pragma unroll
    for (int i = 0; i < 9; i++) dw[i] = lds_u32(a + 4 * i);
    float acc[M];
#pragma unroll
    for (int j = 0; j < M; j++) acc[j] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const u32 q = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float w = (float) (i8) (q >> (8 * k));
#pragma unroll
            for (int j = 0; j < M; j++) acc[j] = __builtin_fmaf(w, x[4 * i + k][j], acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < M; j++) out[j] = d * acc[j];
}

__shared__ u32 sz_iq3s_grid[512];

// The signs of four weights (bits 0..3 of n) applied to their packed magnitudes (four bytes, each at most 15): a set bit
// negates its byte.  n * 0x00204081 puts bit i of n at bit 8 i (and others in between), the mask leaves 0 or 1 a byte, times 255 is
// 0x00 or 0xff a byte, and (m ^ ff) + 1 = -m byte by byte (no carries: the magnitudes are below 128, and -m + ... stays in its byte).
__device__ __forceinline__ u32 iq3s_signed4(u32 mags, u32 n) {
    const u32 one = (n * 0x00204081u) & 0x01010101u;
    return (mags ^ (one * 255u)) + one;
}

template <int M>
__device__ __forceinline__ void unit_dot_iq3_s(u32 o, u32 u, const float (&x)[32][M], float (&out)[M]) {
    const u32 b = o + 110 * (u >> 3), g = u & 7;
    const float d = f16_to_f32((u16) lds_u16(b));
    const u32 qo = b + 2 + 8 * g;
    const u32 qs0 = lds_u16(qo) | (lds_u16(qo + 2) << 16), qs1 = lds_u16(qo + 4) | (lds_u16(qo + 6) << 16);
    const u32 qh = lds_u8(b + 66 + g);
    const u32 so = b + 74 + 4 * g;
    const u32 signs = lds_u16(so) | (lds_u16(so + 2) << 16);
    const u32 sc = (lds_u8(b + 106 + (g >> 1)) >> (4 * (g & 1))) & 0x0f;
    const float db = d * (float) (1 + 2 * sc);
    float acc[M];
#pragma unroll
    for (int j = 0; j < M; j++) acc[j] = 0.0f;
#pragma unroll
    for (int jj = 0; jj < 8; jj++) {
        // the table's byte offset: 4 * (index byte | high bit << 8), from two bit-field extracts, a shift and a shift-or
        const u32 at = (__builtin_amdgcn_ubfe(jj < 4 ? qs0 : qs1, 8 * (jj & 3), 8) << 2) | (__builtin_amdgcn_ubfe(qh, jj, 1) << 10);
        const u32 grid = *(const u32*) ((const u8*) sz_iq3s_grid + at);
        const u32 sg = iq3s_signed4(grid, __builtin_amdgcn_ubfe(signs, 4 * jj, 4));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = 4 * jj + k;
            const float w = (float) (i8) (sg >> (8 * k));        // one sign-extending byte conversion
#pragma unroll
            for (int j = 0; j < M; j++) acc[j] = __builtin_fmaf(w, x[i][j], acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < M; j++) out[j] = db * acc[j];
}

template <class F, int M>
__device__ __forceinline__ void unit_dot(u32 o, u32 u, const float (&x)[32][M], float (&out)[M]) {
    if constexpr (F::BB == 34) unit_dot_q8_0<M>(o, u, x, out);
    else unit_dot_iq3_s<M>(o, u, x, out);
}

// An input row shared by a workgroup through LDS: the 32 inputs of unit u start at float 36 u
// (a lane reads them with eight 16-byte LDS loads; the 4 floats of padding spread the units over the banks).  Reading a
// unit's 128 bytes from global memory lane by lane instead costs the texture path a cache line a lane per load.
constexpr u32 XU_PITCH = 36;

__device__ __forceinline__ void unit_from_lds(const float* xs, u32 u, float (&x)[32][1]) {
    const f32x4* p = (const f32x4*) (xs + u * XU_PITCH);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 v = p[i];
        x[4 * i][0] = v.x;
        x[4 * i + 1][0] = v.y;
        x[4 * i + 2][0] = v.z;
        x[4 * i + 3][0] = v.w;
    }
}

// ---------------------------------------------------------------------------------------------------- the row kernel
// rows_body for rows of more than 64 units (rpb <= 16: at most 4 rows a wave).  The inputs come in column chunks of 64
// units: the workgroup brings chunk c of every input into LDS (s_in, as for short rows), every lane takes its unit of
// it into registers and adds the unit's product to the running sums of the wave's rows, chunk after chunk in column order.
template <class F, int M, class After>
__device__ __forceinline__ void rows_wide(const u8* __restrict__ w, u32 rows, u32 cols, u32 rpb, const float* (&xp)[M], float* (&yp)[M],
                                          float* res, After after_chunk, float (*s_in)[64 * XU_PITCH]) {
    const u32 tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const u32 rb = cols / F::QK * F::BB, U = cols / 32, NC = (U + 63) / 64;
    const u32 nchunks = (rows + rpb - 1) / rpb;
    for (u32 chunk = blockIdx.x; chunk < nchunks; chunk += gridDim.x) {
        const u32 r0 = chunk * rpb;
        const u32 nrows = min(rpb, rows - r0);
        const u32 head = stage_span(w + (u64) r0 * rb, nrows * rb, tid);
        float tot[4][M];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int j = 0; j < M; j++) tot[r][j] = 0.0f;
        for (u32 c = 0; c < NC; c++) {
            f32x4 piece[M][2];
#pragma unroll
            for (int j = 0; j < M; j++)
#pragma unroll
                for (int h = 0; h < 2; h++) piece[j][h] = ((const f32x4*) xp[j])[min(c * 512 + tid + 256 * h, cols / 4 - 1)];
            if (c) __syncthreads();               // every lane has taken its unit of the chunk before
#pragma unroll
            for (int j = 0; j < M; j++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const u32 i = tid + 256 * h;
                    *(f32x4*) (s_in[j] + (i / 8) * XU_PITCH + (i % 8) * 4) = piece[j][h];
                }
            __syncthreads();                      // the chunk (and, the first time, the staged rows)
            const u32 un = c * 64 + lane;
            if (un < U) {
                float x[32][M];
#pragma unroll
                for (int j = 0; j < M; j++) {
                    const f32x4* p = (const f32x4*) (s_in[j] + lane * XU_PITCH);
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const f32x4 v = p[i];
                        x[4 * i][j] = v.x;
                        x[4 * i + 1][j] = v.y;
                        x[4 * i + 2][j] = v.z;
                        x[4 * i + 3][j] = v.w;
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const u32 lr = wave + 4 * r;
                    if (lr < nrows) {
                        float part[M];
                        unit_dot<F, M>(head + lr * rb, un, x, part);
#pragma unroll
                        for (int j = 0; j < M; j++) tot[r][j] += part[j];
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const u32 lr = wave + 4 * r;
#pragma unroll
            for (int j = 0; j < M; j++) tot[r][j] = seg_sum<64>(tot[r][j], lane);
            if (lane == 0 && lr < nrows) {
#pragma unroll
                for (int j = 0; j < M; j++) {
                    if (yp[j]) yp[j][r0 + lr] = tot[r][j];
                    if (res) res[lr * 4 + j] = tot[r][j];
                }
            }
        }
        __syncthreads();          // every wave is done with the staged bytes and the inputs (and res is complete)
        if (res) {
            after_chunk(r0, nrows);
            __syncthreads();
        }
    }
}

// Row chunks blockIdx.x, blockIdx.x + gridDim.x, .. (rpb rows each) of `w` against M inputs: the inputs are read into
// registers once per workgroup, then every chunk is staged and decoded.  Results go through yp to global memory and, when
// `res` is given, to res[local row * 4 + j] in LDS, after which after_chunk(first row, rows) runs on every thread between
// two barriers.  cols is a multiple of 32 (and of the format's block).
template <class F, int M, class After>
__device__ __forceinline__ void rows_body(const u8* __restrict__ w, u32 rows, u32 cols, u32 rpb, const float* (&xp)[M],
                                          float* (&yp)[M], float* res, After after_chunk) {
    const u32 tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const u32 rb = cols / F::QK * F::BB;
    if constexpr (F::BB == 110) {
        for (u32 i = tid; i < 512; i += 256) sz_iq3s_grid[i] = IQ3S_GRID[i];
    }
    const u32 U = cols / 32;
    u32 UL = 64;                          // lanes a row takes in a wave: the units of a row of fewer than 64, rounded up to a power of two
    if (U < 64) {
        UL = 1;
        while (UL < U) UL *= 2;
    }
    const u32 RG = 64 / UL;               // rows side by side in a wave
    const u32 NC = (U + UL - 1) / UL;     // column chunks of UL units; lanes past the row's last unit add nothing
    const u32 sub = lane / UL, ul = lane % UL;
    float x[32][M];
    // the workgroup reads the inputs with whole-line loads and hands them out through LDS
    __shared__ __attribute__((aligned(16))) float s_in[M][64 * XU_PITCH];
    if (NC != 1) {
        rows_wide<F, M>(w, rows, cols, rpb, xp, yp, res, after_chunk, s_in);
        return;
    }
    f32x4 piece[M][2];
#pragma unroll
    for (int j = 0; j < M; j++)
#pragma unroll
        for (int h = 0; h < 2; h++) piece[j][h] = ((const f32x4*) xp[j])[min(tid + 256 * h, cols / 4 - 1)];
    bool first = true;
    const u32 nchunks = (rows + rpb - 1) / rpb;
    for (u32 chunk = blockIdx.x; chunk < nchunks; chunk += gridDim.x) {
        const u32 r0 = chunk * rpb;
        const u32 nrows = min(rpb, rows - r0);
        const u32 head = stage_span(w + (u64) r0 * rb, nrows * rb, tid);
        if (first) {
#pragma unroll
            for (int j = 0; j < M; j++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const u32 i = tid + 256 * h;
                    if (i < cols / 4) *(f32x4*) (s_in[j] + (i / 8) * XU_PITCH + (i % 8) * 4) = piece[j][h];
                }
        }
        __syncthreads();
        if (first) {
            first = false;
#pragma unroll
            for (int j = 0; j < M; j++) {
                const f32x4* p = (const f32x4*) (s_in[j] + ul * XU_PITCH);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const f32x4 v = p[i];
                    x[4 * i][j] = v.x;
                    x[4 * i + 1][j] = v.y;
                    x[4 * i + 2][j] = v.z;
                    x[4 * i + 3][j] = v.w;
                }
            }
        }
        for (u32 lr = wave * RG + sub; lr < rpb; lr += 4 * RG) {   // lr < rpb for every lane of a wave alike, or for none
            float tot[M];
#pragma unroll
            for (int j = 0; j < M; j++) tot[j] = 0.0f;
            if (lr < nrows && ul < U) unit_dot<F, M>(head + lr * rb, ul, x, tot);
#pragma unroll
            for (int j = 0; j < M; j++) tot[j] = seg_sum_rt(tot[j], UL, lane);
            if (ul == 0 && lr < nrows) {
#pragma unroll
                for (int j = 0; j < M; j++) {
                    if (yp[j]) yp[j][r0 + lr] = tot[j];
                    if (res) res[lr * 4 + j] = tot[j];
                }
            }
        }
        __syncthreads();          // every wave is done with the staged bytes (and res is complete)
        if (res) {
            after_chunk(r0, nrows);
            __syncthreads();
        }
    }
}

struct NoAfter {
    __device__ __forceinline__ void operator()(u32, u32) const {}
};

template <class F, class After>
__device__ __forceinline__ void rows_dispatch(const u8* w, u32 rows, u32 cols, u32 rpb, u32 n, const float* (&xp)[4],
                                              float* (&yp)[4], float* res, After after) {
    if (n == 1) {
        const float* x1[1] = {xp[0]};
        float* y1[1] = {yp[0]};
        rows_body<F, 1>(w, rows, cols, rpb, x1, y1, res, after);
    } else if (n == 2) {
        const float* x2[2] = {xp[0], xp[1]};
        float* y2[2] = {yp[0], yp[1]};
        rows_body<F, 2>(w, rows, cols, rpb, x2, y2, res, after);
    } else if (n >= 3) {
        rows_body<F, 4>(w, rows, cols, rpb, xp, yp, res, after);
    }
}

// y_j = W x_j for inputs j = 4 blockIdx.y .. +4 (< m): x rows xs floats apart, y rows ys apart (matvec.cu:677-756).
// grid = (ceil(rows / rpb), ceil(m / 4)), block 256, dynamic LDS = rpb * row bytes + 32.
template <class F>
__device__ __forceinline__ void cols_kernel(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows, u32 cols, u32 m, u32 rpb) {
    const u32 j0 = blockIdx.y * 4;
    const u32 n = min(4u, m - j0);
    const float* xp[4];
    float* yp[4];
    for (u32 j = 0; j < 4; j++) {
        const u32 jj = j0 + (j < n ? j : 0);
        xp[j] = x + (u64) jj * xs;
        yp[j] = j < n ? y + (u64) jj * ys : nullptr;
    }
    rows_dispatch<F>(w, rows, cols, rpb, n, xp, yp, nullptr, NoAfter());
}

extern "C" __global__ void __launch_bounds__(256) matvec_cols_q8_0(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows,
                                                                   u32 cols, u32 m, u32 rpb) {
    cols_kernel<Q80>(w, x, xs, y, ys, rows, cols, m, rpb);
}

extern "C" __global__ void __launch_bounds__(256) matvec_cols_iq3_s(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows,
                                                                    u32 cols, u32 m, u32 rpb) {
    cols_kernel<IQ3S>(w, x, xs, y, ys, rows, cols, m, rpb);
}

// Group g = blockIdx.y: matrix wtab[g] (device address), record gtab[17 g] = {n <= 4 (0: unused slot), xi[8], yi[8]};
// y[yi[j]] = W x[xi[j]] (matvec.cu:1576-1677).  grid = (ceil(rows / rpb), groups).
template <class F>
__device__ __forceinline__ void grouped_kernel(const u64* wtab, const u32* gtab, const float* x, u32 xs, float* y, u32 ys, u32 rows,
                                               u32 cols, u32 rpb) {
    const u32* rec = gtab + 17 * (u64) blockIdx.y;
    const u32 n = min(rec[0], 4u);
    if (n == 0) return;
    const u8* w = (const u8*) wtab[blockIdx.y];
    const float* xp[4];
    float* yp[4];
    for (u32 j = 0; j < 4; j++) {
        const u32 jj = j < n ? j : 0;
        xp[j] = x + (u64) rec[1 + jj] * xs;
        yp[j] = j < n ? y + (u64) rec[9 + jj] * ys : nullptr;
    }
    rows_dispatch<F>(w, rows, cols, rpb, n, xp, yp, nullptr, NoAfter());
}

extern "C" __global__ void __launch_bounds__(256) matvec_grouped_q8_0(const u64* wtab, const u32* gtab, const float* x, u32 xs, float* y,
                                                                      u32 ys, u32 rows, u32 cols, u32 rpb) {
    grouped_kernel<Q80>(wtab, gtab, x, xs, y, ys, rows, cols, rpb);
}

extern "C" __global__ void __launch_bounds__(256) matvec_grouped_iq3_s(const u64* wtab, const u32* gtab, const float* x, u32 xs, float* y,
                                                                       u32 ys, u32 rows, u32 cols, u32 rpb) {
    grouped_kernel<IQ3S>(wtab, gtab, x, xs, y, ys, rows, cols, rpb);
}

// Rows [rpb blockIdx.x, +rpb) of w against the workgroup's inputs in LDS, for a launch with one chunk a workgroup and a
// row's units inside a wave (U = cols / 32 divides 64): the sums are those of rows_body with one input, bit for bit.
// Every thread has passed a barrier since xs (and the IQ3_S table) was written.
template <class F>
__device__ __forceinline__ void rows_one_chunk(const u8* w, u32 rows, u32 cols, u32 rpb, u32 head, const float* xs, float* y) {
    const u32 lane = threadIdx.x % 64, wv = threadIdx.x / 64;
    const u32 U = cols / 32, rb = cols / F::QK * F::BB;
    const u32 r0 = blockIdx.x * rpb;
    const u32 nrows = min(rpb, rows - r0);
    const u32 lg = 31u - (u32) __builtin_clz(U), RG = 64u >> lg, sub = lane >> lg, ul = lane & (U - 1);   // U divides 64: a power of two
    float x[32][1];
    unit_from_lds(xs, ul, x);
    for (u32 lr = wv * RG + sub; lr < rpb; lr += 4 * RG) {
        float tot[1] = {0.0f};
        if (lr < nrows) unit_dot<F, 1>(head + lr * rb, ul, x, tot);
        tot[0] = seg_sum_rt(tot[0], U, lane);
        if (ul == 0 && lr < nrows) y[r0 + lr] = tot[0];
    }
}

// -------------------------------------------------------------------------------------- the verify layer, GGUF experts
// A resident Q8_0 / IQ3_S layer for a verify batch (m <= 8 rows) without a plan, in the shape of the EXL3 one: the work
// items are the (token, expert) pairs themselves, one input each: pair p = j k + t of token j and rank t for p < m k, then
// the shared expert's pair m k + j of every token j.  Expert e's three matrices sit at ebase + e estride + {0, part, 2 part}
// (gate, up, down), the shared expert's at shbase + the same offsets (shbase = 0: none).
// pbuf holds u32 tidx[m k] | f32 w[m k] | u32 cnt[m]; eg holds the gate rows [S][ff] then the up rows [S][ff], S = m (k + 1).
// Every product is the single-input case of rows_body, so the numbers are those of the planned path bit for bit.

// Launch 1: routing (every workgroup of a routed pair redoes its token's selection on one of its waves; the workgroups
// with blockIdx.x == 0 of the gate half also publish tidx), then rows [rpb blockIdx.x, +rpb) of gate (sel 0) or up (sel 1).
// grid = (ceil(ff / rpb), 2 S), block 256, dynamic LDS = rpb * row bytes + 32.
template <class F>
__device__ __forceinline__ void verify_gate_up_gguf(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, u8* pbuf,
                                                    float* eg, u32 ne, u32 k, u32 m, u32 hidden, u32 ff, u32 rpb) {
    __shared__ u32 s_top[16];
    __shared__ double s_ex[512];   // only the exact fallback of the routing touches it
    __shared__ __attribute__((aligned(16))) float s_x[64 * XU_PITCH];
    const u32 G = m * k, S = G + m;
    const u32 wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const u32 sel = blockIdx.y / S, pair = blockIdx.y % S;
    const u32 j = pair < G ? pair / k : pair - G;
    const float* xp[1] = {u + (u64) j * hidden};
    float* yp[1] = {eg + (u64) (sel * S + pair) * ff};
    // one chunk a workgroup and a row's units inside a wave: the token's inputs go through LDS, with loads that are asked
    // for before the routing and cost it little (whole lines a wave, unlike a lane's own 128 bytes)
    const u32 U = hidden / 32;
    const bool one = U <= 64 && 64 % U == 0 && gridDim.x * rpb >= ff;
    if (one) {
        for (u32 i = threadIdx.x; i < hidden / 4; i += 256) *(f32x4*) (s_x + (i / 8) * XU_PITCH + (i % 8) * 4) = ((const f32x4*) xp[0])[i];
        if constexpr (F::BB == 110) {
            for (u32 i = threadIdx.x; i < 512; i += 256) sz_iq3s_grid[i] = IQ3S_GRID[i];
        }
    }
    const u8* w;
    if (pair < G) {
        const u32 t = pair % k;
        if (wave == ((blockIdx.x + blockIdx.y) & 3u)) {
            __builtin_amdgcn_s_setprio(3);   // every other wave of the workgroup waits for this one
            route_id_of_rank(logits + (u64) j * ne, ne, k, t, lane, s_ex, s_top);   // only s_top[t] is read
            __builtin_amdgcn_s_setprio(0);
            if (sel == 0 && blockIdx.x == 0 && lane == 0) ((u32*) pbuf)[pair] = s_top[t];
        }
        __syncthreads();
        const u32 e = s_top[t];
        if (e == 0xffffffffu) return;
        w = (const u8*) (ebase + e * estride + (u64) sel * part);
    } else {
        if (!shbase) return;
        w = (const u8*) (shbase + (u64) sel * part);
    }
    if (one) {
        const u32 rb = hidden / F::QK * F::BB, r0 = blockIdx.x * rpb;
        const u32 head = stage_span(w + (u64) r0 * rb, min(rpb, ff - r0) * rb, threadIdx.x);
        __syncthreads();       // the rows, and for the shared expert's pairs also s_x and the table
        rows_one_chunk<F>(w, ff, hidden, rpb, head, s_x, yp[0]);
        return;
    }
    rows_body<F, 1>(w, ff, hidden, rpb, xp, yp, nullptr, NoAfter());
}

// Launch 2: act = silu(gate) * up of the pair (every workgroup makes its own copy in LDS: ff values), then rows
// [rpb blockIdx.x, +rpb) of down into eo[pair][hidden].  One wave a token also computes the routing weights and the count
// for the combine.  grid = (ceil(hidden / rpb), S), block 256, dynamic LDS = rpb * row bytes + 32; ff <= 4096.
template <class F>
__device__ __forceinline__ void verify_down_gguf(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, u8* pbuf, const float* eg,
                                                 float* eo, u32 ne, u32 k, u32 m, u32 hidden, u32 ff, u32 rpb) {
    __shared__ __attribute__((aligned(16))) float act[4096];
    const u32 G = m * k, S = G + m;
    const u32 wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const u32 pair = blockIdx.y;
    if (pair < G && pair % k == 0 && blockIdx.x == 0 && wave == 3) {
        const u32 j = pair / k;
        u32 kk;
        const float wt = route_weights(logits + (u64) j * ne, ne, k, lane, (const u32*) pbuf + pair, &kk);
        if (lane < k) ((float*) (pbuf + G * 4))[pair + lane] = wt;
        if (lane == 0) ((u32*) (pbuf + 2 * G * 4))[j] = kk;
    }
    const u8* w;
    if (pair < G) {
        const u32 e = ((const u32*) pbuf)[pair];
        if (e == 0xffffffffu) return;
        w = (const u8*) (ebase + e * estride + 2 * (u64) part);
    } else {
        if (!shbase) return;
        w = (const u8*) (shbase + 2 * (u64) part);
    }
    const float* g = eg + (u64) pair * ff;
    const float* up = eg + (u64) (S + pair) * ff;
    const float* xp[1] = {act};
    float* yp[1] = {eo + (u64) pair * hidden};
    const u32 U = ff / 32;
    if (ff <= 1024 && U <= 64 && 64 % U == 0 && gridDim.x * rpb >= hidden) {
        // one chunk a workgroup and a row's units inside a wave: the launch-1 sums are requested first, the chunk's rows
        // next, and act is made while the rows are on their way (rows_body would take the two round trips in turn)
        const u32 tid = threadIdx.x;
        float gv[4], uv[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 c = min(tid + 256 * i, ff - 1);
            gv[i] = g[c];
            uv[i] = up[c];
        }
        if constexpr (F::BB == 110) {
            for (u32 i = tid; i < 512; i += 256) sz_iq3s_grid[i] = IQ3S_GRID[i];
        }
        const u32 rb = ff / F::QK * F::BB;
        const u32 r0 = blockIdx.x * rpb;
        const u32 head = stage_span(w + (u64) r0 * rb, min(rpb, hidden - r0) * rb, tid);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 c = tid + 256 * i;
            if (c < ff) act[(c / 32) * XU_PITCH + c % 32] = siluf_ref(gv[i]) * uv[i];
        }
        __syncthreads();
        rows_one_chunk<F>(w, hidden, ff, rpb, head, act, yp[0]);
        return;
    }
    for (u32 i = threadIdx.x; i < ff; i += 256) act[i] = siluf_ref(g[i]) * up[i];
    __syncthreads();
    rows_body<F, 1>(w, hidden, ff, rpb, xp, yp, nullptr, NoAfter());
}

// ------------------------------------------------------------------------ the decode layer (one token) in two launches
// For a single token the down launch can own a row chunk for ALL of the token's experts, weight and add them in rank order
// itself, and the combine launch goes away.  Launch 1 then hands over act = silu(gate) * up instead of the two sums (a
// workgroup takes the same rows of gate and of up), and one wave of it computes the routing weights, which launch 2 only reads.
// pbuf as above; act holds S rows of ff floats.  The sums are rows_body's single-input sums and the combine is
// moe_combine_qwen_rows's arithmetic; the routing weights are ex_t over the sum of the chosen ex (route_weights_chosen), within
// a unit in the last place of the three-launch form's, so y agrees with that form to the last bit or two, not bit for bit.

// floor(x / d) for x < 65536 by one multiplication: `magic` = fast_div_magic(d), 1 <= d < 65536 (the one division, done once).
__device__ __forceinline__ u32 fast_div_magic(u32 d) { return 0xffffffffu / d + 1u; }
__device__ __forceinline__ u32 fast_div(u32 x, u32 magic) { return __umulhi(x, magic); }

// Copies `n` spans of `span` bytes into LDS regions of `rs` bytes each (a multiple of 16, at least span + 15): span p starts
// at global address g0(p) and lands so that its first byte is at byte (g0(p) & 15) of region p, which starts at dynamic LDS
// byte p * rs; a null g0(p) skips the span.  All the loads of a thread (at most 4: n * rs / 16 <= 1024) are in flight
// before its first store; a chunk that reaches outside its span is read byte by byte, so nothing outside the spans is touched.
template <class Addr>
__device__ __forceinline__ void stage_spans(Addr g0, u32 n, u32 span, u32 rs, u32 tid) {
    const u32 ch = rs / 16, total = n * ch, nthr = blockDim.x, mch = fast_div_magic(ch);
    u32x4 v[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const u32 i = tid + nthr * r;
        v[r] = u32x4{0, 0, 0, 0};
        if (i < total) {
            const u32 p = fast_div(i, mch), c = i - p * ch;
            const u8* g = g0(p);
            if (g) {
                const u32 head = (u32) ((u64) g & 15);
                const u8* a0 = g - head;
                const u32 lo = c * 16, end = head + span;
                if (lo >= head && lo + 16 <= end) {
                    v[r] = *(const u32x4*) (a0 + lo);
                } else if (lo < end && lo + 16 > head) {
                    u32 w[4] = {0, 0, 0, 0};
                    for (u32 b = 0; b < 16; b++) {
                        const u32 idx = lo + b;
                        if (idx >= head && idx < end) w[b / 4] |= (u32) a0[idx] << (8 * (b % 4));
                    }
                    v[r] = u32x4{w[0], w[1], w[2], w[3]};
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const u32 i = tid + nthr * r;
        if (i < total) ((u32x4*) sz_dyn_lds)[i] = v[r];
    }
}

// Launch 1: as verify_gate_up_gguf for one chunk a workgroup, but the workgroup takes rows [rp blockIdx.x, +rp) of gate AND
// of up and writes act.  The workgroup blockIdx.x == 0 of every token's last pair (the shared expert's, or rank 0's when
// there is none) also selects all k experts on a wave of its own and leaves ids, weights and count in pbuf.
// grid = (ff / rp, S), block 256 to 1024 (a wave takes the rows wave, wave + waves, ..), dynamic LDS = 2 * (rp * row bytes + 32); hidden / 32 divides 64, rp divides ff.
template <class F>
__device__ __forceinline__ void decode_gate_up_gguf(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, u8* pbuf,
                                                    float* act, u32 ne, u32 k, u32 m, u32 hidden, u32 ff, u32 rp) {
    __shared__ u32 s_top[16], s_all[16];
    __shared__ double s_ex[512], s_ex_all[512];   // only the exact fallback of the routing touches them
    __shared__ __attribute__((aligned(16))) float s_x[64 * XU_PITCH];
    const u32 G = m * k, S = G + m;
    const u32 wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const u32 pair = blockIdx.y;
    const u32 j = pair < G ? pair / k : pair - G;
    if (pair >= G && !shbase) return;
    for (u32 i = threadIdx.x; i < hidden / 4; i += blockDim.x) *(f32x4*) (s_x + (i / 8) * XU_PITCH + (i % 8) * 4) = ((const f32x4*) (u + (u64) j * hidden))[i];
    if constexpr (F::BB == 110) {
        for (u32 i = threadIdx.x; i < 512; i += blockDim.x) sz_iq3s_grid[i] = IQ3S_GRID[i];
    }
    const u32 rwave = (blockIdx.x + blockIdx.y) & 3u;             // the wave that finds this pair's expert
    const bool all = blockIdx.x == 0 && pair == (shbase ? G + j : j * k);
    if (all && wave == ((rwave + 1) & 3u)) {
        const float* lg = logits + (u64) j * ne;
        __builtin_amdgcn_s_setprio(3);
        route_ids(lg, ne, k, lane, s_ex_all, s_all);
        u32 kk;
        const float wt = route_weights_chosen(lg, ne, k, lane, s_all, &kk);
        if (lane < k) {
            ((u32*) pbuf)[j * k + lane] = s_all[lane];
            ((float*) (pbuf + G * 4))[j * k + lane] = wt;
        }
        if (lane == 0) ((u32*) (pbuf + 2 * G * 4))[j] = kk;
        __builtin_amdgcn_s_setprio(0);
    }
    const u8* w;
    if (pair < G) {
        const u32 t = pair % k;
        if (wave == rwave) {
            // the wave every other wave of the workgroup waits for: it goes first where it shares a SIMD with waves of
            // workgroups that are already multiplying
            __builtin_amdgcn_s_setprio(3);
            route_id_of_rank(logits + (u64) j * ne, ne, k, t, lane, s_ex, s_top);   // only s_top[t] is read
            __builtin_amdgcn_s_setprio(0);
        }
        __syncthreads();
        const u32 e = s_top[t];
        if (e == 0xffffffffu) return;
        w = (const u8*) (ebase + e * estride);
    } else {
        w = (const u8*) shbase;
    }
    const u32 rb = hidden / F::QK * F::BB, r0 = blockIdx.x * rp;
    const u32 rs = (rp * rb + 31) / 16 * 16;
    stage_spans([&](u32 p) { return w + (u64) p * part + (u64) r0 * rb; }, 2, rp * rb, rs, threadIdx.x);
    __syncthreads();       // the rows, and for the shared expert's pairs also s_x and the table
    const u32 hg = (u32) ((u64) (w + (u64) r0 * rb) & 15), hu = rs + (u32) ((u64) (w + (u64) part + (u64) r0 * rb) & 15);
    const u32 U = hidden / 32, lg = 31u - (u32) __builtin_clz(U), RG = 64u >> lg, sub = lane >> lg, ul = lane & (U - 1);   // U divides 64: a power of two
    float x[32][1];
    unit_from_lds(s_x, ul, x);
    float* o = act + (u64) pair * ff + r0;
    for (u32 lr = wave * RG + sub; lr < rp; lr += (blockDim.x / 64) * RG) {
        float g[1] = {0.0f}, up[1] = {0.0f};
        unit_dot<F, 1>(hg + lr * rb, ul, x, g);
        unit_dot<F, 1>(hu + lr * rb, ul, x, up);
        g[0] = seg_sum_rt(g[0], U, lane);
        up[0] = seg_sum_rt(up[0], U, lane);
        if (ul == 0) o[lr] = siluf_ref(g[0]) * up[0];
    }
}

// Launch 2 for one token: rows [rd blockIdx.x, +rd) of the down matrix of every chosen expert and of the shared one against
// that pair's act, then y = the sum in rank order of weight * row, plus sigmoid(gate logit) * the shared expert's row.
// grid = hidden / rd, block 256 to 1024 (a wave takes the pairs wave, wave + waves, ..), dynamic LDS = S * region + S * (ff / 32) * 144 with region = rd * row bytes + 31 rounded
// down to 16; ff / 32 divides 64, 64 / (ff / 32) divides rd, rd divides hidden, S * region <= 16 KiB, S * ff <= 8192, k <= 16.
template <class F>
__device__ __forceinline__ void decode_down_combine_gguf(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf, const float* act,
                                                         const float* gl, float* y, u32 k, u32 hidden, u32 ff, u32 rd) {
    __shared__ float s_eo[17][64];
    __shared__ float s_w[16];
    const u32 G = k, S = shbase ? k + 1 : k;
    const u32 tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const u32 rb = ff / F::QK * F::BB, r0 = blockIdx.x * rd;
    const u32 rs = (rd * rb + 31) / 16 * 16;
    const u32 U = ff / 32, nthr = blockDim.x;
    float* s_act = (float*) ((u8*) sz_dyn_lds + S * rs);
    // every load goes out before anything is waited for: the pairs' act, the chosen ids, then the rows
    const u32 n4 = ff / 4, pieces = S * n4;
    f32x4 av[8];
#pragma unroll
    for (int h = 0; h < 8; h++) av[h] = ((const f32x4*) act)[min(tid + nthr * h, pieces - 1)];
    const u32 myid = ((const u32*) pbuf)[min(lane, k - 1)];
    const float wt = ((const float*) (pbuf + G * 4))[min(lane, k - 1)];
    const u32 cnt = ((const u32*) (pbuf + 2 * G * 4))[0];
    const float glv = shbase ? gl[0] : 0.0f;
    if constexpr (F::BB == 110) {
        for (u32 i = tid; i < 512; i += nthr) sz_iq3s_grid[i] = IQ3S_GRID[i];
    }
    if (wave == 0 && lane < 16) s_w[lane] = lane < k ? wt : 0.0f;
    // the experts' addresses need the ids, which every wave holds in its lanes 0..k-1: a wave-level broadcast
    auto row_of = [&](u32 p) -> const u8* {
        if (p >= G) return (const u8*) (shbase + 2 * (u64) part + (u64) r0 * rb);
        const u32 e = (u32) __shfl((int) myid, (int) p, SZ_WAVE);
        return e == 0xffffffffu ? nullptr : (const u8*) (ebase + e * estride + 2 * (u64) part + (u64) r0 * rb);
    };
    // as stage_spans, with every lane fetching the id of its chunk's pair from the lane that holds it
    {
        const u32 ch = rs / 16, total = S * ch, mch = fast_div_magic(ch), mn4 = fast_div_magic(n4);
        u32x4 v[4];
        const u8* src[4];
        u32 lo[4], hd[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const u32 i = min(tid + nthr * r, total - 1), p = fast_div(i, mch);
            const u8* g = nullptr;
            // (p differs between the lanes of a wave: every lane fetches its pair's id from the lane that holds it)
            if (p >= G) g = (const u8*) (shbase + 2 * (u64) part + (u64) r0 * rb);
            const u32 e = (u32) __shfl((int) myid, (int) min(p, k - 1), SZ_WAVE);
            if (p < G && e != 0xffffffffu) g = (const u8*) (ebase + e * estride + 2 * (u64) part + (u64) r0 * rb);
            src[r] = g;
            hd[r] = (u32) ((u64) g & 15);
            lo[r] = (i - p * ch) * 16;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            v[r] = u32x4{0, 0, 0, 0};
            const u32 i = tid + nthr * r;
            if (i < total && src[r]) {
                const u8* a0 = src[r] - hd[r];
                const u32 end = hd[r] + rd * rb;
                if (lo[r] >= hd[r] && lo[r] + 16 <= end) {
                    v[r] = *(const u32x4*) (a0 + lo[r]);
                } else if (lo[r] < end && lo[r] + 16 > hd[r]) {
                    u32 w[4] = {0, 0, 0, 0};
                    for (u32 b = 0; b < 16; b++) {
                        const u32 idx = lo[r] + b;
                        if (idx >= hd[r] && idx < end) w[b / 4] |= (u32) a0[idx] << (8 * (b % 4));
                    }
                    v[r] = u32x4{w[0], w[1], w[2], w[3]};
                }
            }
        }
#pragma unroll
        for (int h = 0; h < 8; h++) {
            const u32 i = tid + nthr * h;
            if (i < pieces) {
                const u32 p = fast_div(i, mn4), q = i - p * n4;
                *(f32x4*) (s_act + (p * U + q / 8) * XU_PITCH + (q % 8) * 4) = av[h];
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const u32 i = tid + nthr * r;
            if (i < total) ((u32x4*) sz_dyn_lds)[i] = v[r];
        }
    }
    __syncthreads();
    const u32 lg = 31u - (u32) __builtin_clz(U), RG = 64u >> lg, sub = lane >> lg, ul = lane & (U - 1);   // U divides 64: a power of two
    for (u32 p = wave; p < S; p += nthr / 64) {
        const u8* g = row_of(p);
        if (!g) continue;                       // a masked rank: nothing was staged and nothing is added
        const u32 head = p * rs + (u32) ((u64) g & 15);
        float x[32][1];
        unit_from_lds(s_act + p * U * XU_PITCH, ul, x);
        for (u32 lr = sub; lr < rd; lr += RG) {
            float tot[1] = {0.0f};
            unit_dot<F, 1>(head + lr * rb, ul, x, tot);
            tot[0] = seg_sum_rt(tot[0], U, lane);
            if (ul == 0) s_eo[p][lr] = tot[0];
        }
    }
    __syncthreads();
    if (tid < rd) {
        float acc = 0.0f;
        for (u32 t = 0; t < k; t++)
            if (t < cnt) acc += s_w[t] * s_eo[t][tid];
        if (shbase) acc += sigmoidf_ref(glv) * s_eo[G][tid];
        y[r0 + tid] = acc;
    }
}

extern "C" __global__ void __launch_bounds__(1024) decode_gate_up_q8_0(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                                      const float* u, u8* pbuf, float* act, u32 ne, u32 k, u32 m, u32 hidden,
                                                                      u32 ff, u32 rp) {
    decode_gate_up_gguf<Q80>(logits, ebase, estride, shbase, part, u, pbuf, act, ne, k, m, hidden, ff, rp);
}
extern "C" __global__ void __launch_bounds__(1024) decode_gate_up_iq3_s(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                                       const float* u, u8* pbuf, float* act, u32 ne, u32 k, u32 m, u32 hidden,
                                                                       u32 ff, u32 rp) {
    decode_gate_up_gguf<IQ3S>(logits, ebase, estride, shbase, part, u, pbuf, act, ne, k, m, hidden, ff, rp);
}
extern "C" __global__ void __launch_bounds__(1024) decode_down_combine_q8_0(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf,
                                                                           const float* act, const float* gl, float* y, u32 k, u32 hidden,
                                                                           u32 ff, u32 rd) {
    decode_down_combine_gguf<Q80>(ebase, estride, shbase, part, pbuf, act, gl, y, k, hidden, ff, rd);
}
extern "C" __global__ void __launch_bounds__(1024) decode_down_combine_iq3_s(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf,
                                                                            const float* act, const float* gl, float* y, u32 k, u32 hidden,
                                                                            u32 ff, u32 rd) {
    decode_down_combine_gguf<IQ3S>(ebase, estride, shbase, part, pbuf, act, gl, y, k, hidden, ff, rd);
}

extern "C" __global__ void __launch_bounds__(256) verify_gate_up_q8_0(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                                      const float* u, u8* pbuf, float* eg, u32 ne, u32 k, u32 m, u32 hidden,
                                                                      u32 ff, u32 rpb) {
    verify_gate_up_gguf<Q80>(logits, ebase, estride, shbase, part, u, pbuf, eg, ne, k, m, hidden, ff, rpb);
}

extern "C" __global__ void __launch_bounds__(256) verify_down_q8_0(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, u8* pbuf,
                                                                   const float* eg, float* eo, u32 ne, u32 k, u32 m, u32 hidden, u32 ff,
                                                                   u32 rpb) {
    verify_down_gguf<Q80>(logits, ebase, estride, shbase, part, pbuf, eg, eo, ne, k, m, hidden, ff, rpb);
}

extern "C" __global__ void __launch_bounds__(256) verify_gate_up_iq3_s(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                                      const float* u, u8* pbuf, float* eg, u32 ne, u32 k, u32 m, u32 hidden,
                                                                      u32 ff, u32 rpb) {
    verify_gate_up_gguf<IQ3S>(logits, ebase, estride, shbase, part, u, pbuf, eg, ne, k, m, hidden, ff, rpb);
}

extern "C" __global__ void __launch_bounds__(256) verify_down_iq3_s(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, u8* pbuf,
                                                                   const float* eg, float* eo, u32 ne, u32 k, u32 m, u32 hidden, u32 ff,
                                                                   u32 rpb) {
    verify_down_gguf<IQ3S>(logits, ebase, estride, shbase, part, pbuf, eg, eo, ne, k, m, hidden, ff, rpb);
}

// ------------------------------------------------------------------------------- unquantized matrices (F32, F16, BF16)
// The router, the shared expert's gate and the other small projections are stored unquantized (quant.rs:237-239).  One wave
// a row: a lane takes 4 consecutive columns a step (one 16- or 8-byte load), 256 columns a step for the wave, the row's
// products are added in f32 lane by lane and then over the wave; every input of the batch (m <= 8) reuses the loaded
// weights.  cols is a multiple of 4, rows of x are 16-byte aligned, rows of w are aligned to 4 weights, rows >= 1.
struct DenseF32 {
    static constexpr u32 BYTES = 4;
    static __device__ __forceinline__ f32x4 load4(const u8* p) { return *(const f32x4*) p; }
};
struct DenseF16 {
    static constexpr u32 BYTES = 2;
    static __device__ __forceinline__ f32x4 load4(const u8* p) {
        const uint2 v = *(const uint2*) p;
        return f32x4{f16_to_f32((u16) v.x), f16_to_f32((u16) (v.x >> 16)), f16_to_f32((u16) v.y), f16_to_f32((u16) (v.y >> 16))};
    }
};
struct DenseBF16 {
    static constexpr u32 BYTES = 2;
    static __device__ __forceinline__ f32x4 load4(const u8* p) {   // half.rs: a bf16 is the upper half of the f32
        const uint2 v = *(const uint2*) p;
        return f32x4{bits_f32(v.x << 16), bits_f32(v.x & 0xffff0000u), bits_f32(v.y << 16), bits_f32(v.y & 0xffff0000u)};
    }
};

// What a job does to a finished product t: 0 nothing; 1 silu(t / div); 2 2 sigmoid(t / div); 3 sigmoid(t) - the
// hyper-connection's down, inject and up projections (forward.rs:804-814).
__device__ __forceinline__ float dense_act(float t, u32 act, float div) {
    if (act == 1) return siluf_ref(t / div);
    if (act == 2) return 2.0f * sigmoidf_ref(t / div);
    if (act == 3) return sigmoidf_ref(t);
    return t;
}

#define DENSE_CHUNK 2048u   // columns a wave takes at a time: 8 loads of 4 a lane
// rows a wave takes in turn when the rows are short: up to 8, fewer while that would leave CUs without a workgroup
__device__ __forceinline__ u32 dense_rpw(u32 rows) { return min(8u, max(1u, rows / 1024u)); }

// The wave's weights of columns [c0, c0 + chunk) of the row at wr, 4 a lane a load, all 8 loads in flight together.
template <class T>
__device__ __forceinline__ void dense_load_w(const u8* __restrict__ wr, u32 c0, u32 chunk, bool live, u32 lane, f32x4 (&wv)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const u32 c = 4 * lane + 256 * i;
        wv[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (live && c < chunk) wv[i] = T::load4(wr + (u64) (c0 + c) * T::BYTES);
    }
}

__device__ __forceinline__ float dense_dot8(const f32x4 (&wv)[8], const f32x4 (&xv)[8], float acc) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc = __builtin_fmaf(wv[i].x, xv[i].x, acc);
        acc = __builtin_fmaf(wv[i].y, xv[i].y, acc);
        acc = __builtin_fmaf(wv[i].z, xv[i].z, acc);
        acc = __builtin_fmaf(wv[i].w, xv[i].w, acc);
    }
    return acc;
}

// Long rows (cols > 2048): one row a workgroup, wave v takes the chunks v, v + 4, .. of it; the inputs' chunks come
// straight from memory (they are shared by every workgroup and stay in cache), an input at a time; the four waves' sums
// are added in wave order.  `row` < rows for every workgroup that calls it.
template <class T>
__device__ __forceinline__ void dense_wide(const u8* __restrict__ w, const float* __restrict__ x, u32 xs, float* __restrict__ y, u32 ys, u32 row,
                                           u32 cols, u32 m, u32 act, float div) {
    float (*red)[8] = (float (*)[8]) sz_dyn_lds;   // 4 x 8 floats of dynamic LDS
    const u32 tid = threadIdx.x, lane = tid % 64, wv_ = tid / 64;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = 0.0f;
    const u8* wr = w + (u64) row * cols * T::BYTES;
    for (u32 c0 = wv_ * DENSE_CHUNK; c0 < cols; c0 += 4 * DENSE_CHUNK) {
        const u32 chunk = min(DENSE_CHUNK, cols - c0);
        f32x4 wv[8];
        dense_load_w<T>(wr, c0, chunk, true, lane, wv);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if ((u32) j < m) {
                f32x4 xv[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const u32 c = 4 * lane + 256 * i;
                    xv[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    if (c < chunk) xv[i] = *(const f32x4*) (x + (u64) j * xs + c0 + c);
                }
                acc[j] = dense_dot8(wv, xv, acc[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        if ((u32) j < m) {
            const float t = seg_sum<64>(acc[j], lane);
            if (lane == 0) red[wv_][j] = t;
        }
    }
    __syncthreads();
    if (tid < m) y[(u64) tid * ys + row] = dense_act(((red[0][tid] + red[1][tid]) + red[2][tid]) + red[3][tid], act, div);
}

// Short rows (cols <= 2048): the inputs are staged into LDS once a workgroup (xl: m * cols floats of dynamic LDS), then
// wave v takes rows r0 + v, r0 + v + 4, .. (rpw of them), the next row's weights on their way while this one is
// multiplied.  Lane 0 writes y[j * ys + row].
template <class T>
__device__ __forceinline__ void dense_narrow(const u8* __restrict__ w, const float* __restrict__ x, u32 xs, float* __restrict__ y, u32 ys, u32 r0,
                                             u32 rpw, u32 rows, u32 cols, u32 m, u32 act, float div) {
    float* xl = (float*) sz_dyn_lds;
    const u32 tid = threadIdx.x, lane = tid % 64, wv_ = tid / 64;
    const u32 q4 = cols / 4, total = m * q4;   // 16-byte pieces of the inputs: at most 16 a thread
    f32x4 wv[8], wn[8];
    u32 row = r0 + wv_;
    dense_load_w<T>(w + (u64) min(row, rows - 1) * cols * T::BYTES, 0, cols, row < rows, lane, wv);
    {
        f32x4 t[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const u32 idx = tid + 256 * i;
            if (idx < total) t[i] = *(const f32x4*) (x + (u64) (idx / q4) * xs + 4 * (idx % q4));
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const u32 idx = tid + 256 * i;
            if (idx < total) *(f32x4*) (xl + (idx / q4) * cols + 4 * (idx % q4)) = t[i];
        }
    }
    __syncthreads();
#pragma unroll 1
    for (u32 it = 0; it < rpw; it++, row += 4) {
        if (row >= rows) break;   // the same for every lane of the wave
        const u32 next = row + 4;
        if (it + 1 < rpw) dense_load_w<T>(w + (u64) min(next, rows - 1) * cols * T::BYTES, 0, cols, next < rows, lane, wn);
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            acc[j] = 0.0f;
            if ((u32) j < m) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const u32 c = 4 * lane + 256 * i;
                    if (c < cols) {
                        const f32x4 xv = *(const f32x4*) (xl + j * cols + c);
                        acc[j] = __builtin_fmaf(wv[i].x, xv.x, acc[j]);
                        acc[j] = __builtin_fmaf(wv[i].y, xv.y, acc[j]);
                        acc[j] = __builtin_fmaf(wv[i].z, xv.z, acc[j]);
                        acc[j] = __builtin_fmaf(wv[i].w, xv.w, acc[j]);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if ((u32) j < m) {
                const float t = seg_sum<64>(acc[j], lane);
                if (lane == 0) y[(u64) j * ys + row] = dense_act(t, act, div);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) wv[i] = wn[i];
    }
}

// Workgroups a matrix of `rows` rows needs: one a row when the rows are long, one for every 4 * dense_rpw(rows) rows otherwise.
// Workgroup g (counted from the matrix's first) of the launch:
template <class T>
__device__ __forceinline__ void dense_group(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows, u32 cols, u32 m, u32 g, u32 act,
                                            float div) {
    if (cols > DENSE_CHUNK) {
        if (g < rows) dense_wide<T>(w, x, xs, y, ys, g, cols, m, act, div);
    } else {
        const u32 rpw = dense_rpw(rows);
        dense_narrow<T>(w, x, xs, y, ys, g * 4 * rpw, rpw, rows, cols, m, act, div);
    }
}

// y_j = W x_j for an unquantized row-major W[rows][cols], j < m <= 8 (matvec_cols_*, kernels/matvec.cu:677).
// cols <= 2048: grid = ceil(rows / (4 * dense_rpw(rows))), dynamic LDS = m * cols * 4; longer rows: grid = rows, dynamic LDS = 128.  block 256.
extern "C" __global__ void __launch_bounds__(256) matvec_cols_f32(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows, u32 cols, u32 m) {
    dense_group<DenseF32>(w, x, xs, y, ys, rows, cols, m, blockIdx.x, 0, 1.0f);
}
extern "C" __global__ void __launch_bounds__(256) matvec_cols_f16(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows, u32 cols, u32 m) {
    dense_group<DenseF16>(w, x, xs, y, ys, rows, cols, m, blockIdx.x, 0, 1.0f);
}
extern "C" __global__ void __launch_bounds__(256) matvec_cols_bf16(const u8* w, const float* x, u32 xs, float* y, u32 ys, u32 rows, u32 cols, u32 m) {
    dense_group<DenseBF16>(w, x, xs, y, ys, rows, cols, m, blockIdx.x, 0, 1.0f);
}

// Several unquantized matrices on the same inputs in one launch (matvec_cols_multi, kernels/matvec.cu:1958: the router and
// the shared expert's gate logit).  jobs[i] = {u64 w, u64 y, u32 ys, u32 rows, u32 type (0 F32, 1 F16, 2 BF16), u32 first, u32 act, f32 div} (dense_act):
// job i owns workgroups [first_i, first_{i+1}), as many as its matrix needs on its own (dense_group); every output is the
// one-matrix kernel's bit for bit.  block 256, dynamic LDS as for one matrix.
struct DenseJob {
    u64 w, y;
    u32 ys, rows, type, first, act;
    float div;
};
extern "C" __global__ void __launch_bounds__(256) matvec_cols_multi(const u8* jobs, u32 njobs, const float* x, u32 xs, u32 cols, u32 m) {
    const DenseJob* jt = (const DenseJob*) jobs;
    u32 i = 0;
    while (i + 1 < njobs && blockIdx.x >= jt[i + 1].first) i++;
    const DenseJob jb = jt[i];
    const u32 g = blockIdx.x - jb.first;
    if (jb.type == 0) dense_group<DenseF32>((const u8*) jb.w, x, xs, (float*) jb.y, jb.ys, jb.rows, cols, m, g, jb.act, jb.div);
    else if (jb.type == 1) dense_group<DenseF16>((const u8*) jb.w, x, xs, (float*) jb.y, jb.ys, jb.rows, cols, m, g, jb.act, jb.div);
    else dense_group<DenseBF16>((const u8*) jb.w, x, xs, (float*) jb.y, jb.ys, jb.rows, cols, m, g, jb.act, jb.div);
}

// ------------------------------------------------------------------------------------------------ lm_head + argmax
// The head product for m <= 4 rows with each workgroup's (maximum, lowest index) of every row over all its row chunks
// written to part[(blockIdx.x * 4 + j) * 2] = {value bits, index}, so the logits never have to be written (logits may be
// null).  A NaN logit counts as -inf, as the device top-k does (kernels/forward.cu:3592).  grid = any number of workgroups up
// to the number of chunks, block 256, dynamic LDS = rpb * row bytes + 32 + rpb * 16.
extern "C" __global__ void __launch_bounds__(256) head_q8_0_argmax(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part,
                                                                   u32 rows, u32 cols, u32 m, u32 rpb) {
    const u32 n = min(4u, m);
    const u32 rb = cols / 32 * 34;
    float* res = (float*) (sz_dyn_lds + (rpb * rb + 32 + 3) / 4);
    const float* xp[4];
    float* yp[4];
    for (u32 j = 0; j < 4; j++) {
        const u32 jj = j < n ? j : 0;
        xp[j] = x + (u64) jj * xs;
        yp[j] = (j < n && logits) ? logits + (u64) jj * ls : nullptr;
    }
    float bv = -__builtin_inff();
    u32 bi = 0xffffffffu;
    const u32 tid = threadIdx.x;
    auto after = [&](u32 r0, u32 nrows) {
        if (tid < n) {
            for (u32 r = 0; r < nrows; r++) {
                float v = res[r * 4 + tid];
                if (v != v) v = -__builtin_inff();
                argmax_merge(bv, bi, v, r0 + r);
            }
        }
    };
    rows_dispatch<Q80>(w, rows, cols, rpb, n, xp, yp, res, after);
    if (tid < n) {
        part[((u64) blockIdx.x * 4 + tid) * 2] = f32_bits(bv);
        part[((u64) blockIdx.x * 4 + tid) * 2 + 1] = bi;
    }
}

// The same head on the matrix cores, for W = 4, 6 or 8 waves and cols <= 512 W (a multiple of 64 W), m <= 8 and a 16-byte aligned matrix.
// A 16-row tile of the matrix (16 x cols / 32 x 34 contiguous bytes) comes into LDS by global-to-LDS loads, the next tile
// while this one is multiplied.  Wave w owns the share k in [w cols / W, (w + 1) cols / W) of every row and keeps its
// slice of the inputs in registers for the whole launch, as the B operands of v_mfma_f32_16x16x16_f16: with
// s_j x_j = the input row times the power of two that takes its largest magnitude to [2^14, 2^15), column 2 j holds
// f16(s_j x_j) and column 2 j + 1 holds f16(s_j x_j - f16(s_j x_j)): the high parts are finite whatever the activations'
// size, the two columns together carry an element to 22 bits unless it is below 2^-17 of the row's largest (there the
// low part runs into f16's subnormals and the element keeps at least its 11 high-part bits, an error below 2^-39 of
// the largest), and every product with the int8 codes (exact in f16) is exact; the matrix core adds in f32 and the sums
// are multiplied by 1 / s_j at the end.  The A operand is the tile's
// codes: a lane takes 4 consecutive codes of row lane % 16, turns each into the f16 1024 + (code ^ 0x80) by putting 0x64
// above the byte, and subtracts 1152 (exact).  A 32-block's two products are scaled by the block's f16 scale and added to
// the lane's running sums in f32, block after block in k order; the waves' sums are added in wave order.
// part[(blockIdx.x * 8 + j) * 2] = {value bits, index} of the workgroup's best row for input j (NaN counts as -inf,
// ties to the lower index).  grid <= tiles (persistent: tile t goes to workgroup t % grid), block 64 W.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
#define HEAD_PITCH(cols) ((cols) / 32 * 34 + 16)   // bytes between a tile's rows in LDS: 16 rows then fall on different banks

__device__ __forceinline__ f16x4 head_codes_f16(u32 q) {
    const u32 u = q ^ 0x80808080u;                                   // code + 128 as unsigned bytes
    const u32 lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);   // halves 0x6400 | byte 0, 0x6400 | byte 1
    const u32 hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
    typedef _Float16 f16x2_ __attribute__((ext_vector_type(2)));
    const f16x2_ k = {(_Float16) -1152.0f, (_Float16) -1152.0f};
    const f16x2_ a = __builtin_bit_cast(f16x2_, lo) + k, b = __builtin_bit_cast(f16x2_, hi) + k;
    return f16x4{a[0], a[1], b[0], b[1]};
}

// Requests tile `t` (rows 16 t .. 16 t + 15, clamped to the last row) into the LDS buffer at byte offset `lds`: wave w of W
// brings rows w, w + W, .., each as 16-byte pieces (ceil(row bytes / 1024) instructions a row).
template <int W>
__device__ __forceinline__ void head_tile_issue(const u8* __restrict__ w, u32 rows, u32 rb, u32 t, u32 lds, u32 wave, u32 lane) {
    const u32 pieces = rb / 16;                           // rb is a multiple of 16 here
#pragma unroll
    for (int rr = 0; rr < (16 + W - 1) / W; rr++) {
        const u32 lr = wave + W * rr;
        if (lr < 16) {
            const u8* src = w + (u64) min(16 * t + lr, rows - 1) * rb;
            const u32 dst = lds + lr * (rb + 16);
#pragma unroll
            for (int c = 0; c < 5; c++)
                if (c * 64 < pieces)
                    if (c * 64 + lane < pieces) lds_load<16>(src + (c * 64 + lane) * 16, dst + c * 1024);
        }
    }
}

// W waves (4, 6 or 8), cols = CMAX (512 W unless a narrower row is given more waves) at most and a multiple of 64 W.
template <int W, int CMAX = 512 * W, bool FULL = false>   // FULL: cols == CMAX, every wave owns NBM blocks (no per-block checks: the tile reads of all blocks go out together)
__device__ __forceinline__ void head_mfma_body(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part, u32 rows, u32 cols, u32 m) {
    __shared__ float s_bv[256];
    __shared__ u32 s_bi[256];
    __shared__ float s_mx[W][8], s_inv[8];   // largest magnitude of a wave's share of every input row; the factor that undoes a row's scale
    const u32 tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    if constexpr (FULL) cols = CMAX;                      // (the host launches this form for no other width: offsets become constants)
    const u32 rb = cols / 32 * 34, pitch = rb + 16;
    constexpr int NBM = CMAX / W / 32;                    // the most 32-blocks a wave owns
    const u32 kw = cols / W, nbw = kw / 32;               // a wave's columns, and their 32-blocks (<= NBM)
    const u32 n16 = lane & 15, g4 = lane >> 4;
    __shared__ __attribute__((aligned(16))) u8 tiles_lds[2 * 16 * HEAD_PITCH(CMAX)];   // two tiles, 16 * pitch bytes apart
    __shared__ float red[W][256];
    u8* const tile0 = tiles_lds;
    // the wave's slice of the inputs as B operands: B[k = 4 g4 + i][n = n16], n = 2 j + (0: high part, 1: low part)
    f16x4 xb[NBM][2];
    {
        const u32 j = n16 >> 1, lowpart = n16 & 1;
        // all 32 loads go out before the first is waited for (clamped to an address that exists where the lane has no
        // input or the block lies past the row: a load behind a branch is waited for on the spot, a round trip each)
        f32x4 raw[NBM][2];
        const float* xj = x + (u64) min(j, m - 1) * xs + wave * kw + 4 * g4;
#pragma unroll
        for (int b = 0; b < NBM; b++)
#pragma unroll
            for (int h = 0; h < 2; h++) raw[b][h] = *(const f32x4*) (xj + 32 * min((u32) b, nbw - 1) + 16 * h);
        // every input row is scaled by a power of two that takes its largest magnitude to [2^14, 2^15) before it is split (the
        // sums are scaled back at the end): the high parts cannot overflow to infinity whatever the activations' size, and
        // the low parts of small activations are not lost to f16's subnormal range
        float mxl = 0.0f;
#pragma unroll
        for (int b = 0; b < NBM; b++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                if (FULL || (u32) b < nbw)
#pragma unroll
                    for (int i = 0; i < 4; i++) mxl = fmaxf(mxl, __builtin_fabsf(raw[b][h][i]));   // a NaN is skipped here and shows in the sums
        mxl = fmaxf(mxl, lane_xor<16>(mxl, lane));
        mxl = fmaxf(mxl, lane_xor<32>(mxl, lane));
        if (g4 == 0 && lowpart == 0) s_mx[wave][j] = mxl;
        __syncthreads();
        float mxr = s_mx[0][j];
#pragma unroll
        for (int v = 1; v < W; v++) mxr = fmaxf(mxr, s_mx[v][j]);
        float scale, inv;
        pow2_scale_of(f32_bits(mxr), scale, inv);
        if (wave == 0 && g4 == 0 && lowpart == 0) s_inv[j] = inv;
#pragma unroll
        for (int b = 0; b < NBM; b++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                f16x4 v = {0, 0, 0, 0};
                if ((FULL || (u32) b < nbw) && j < m) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float f = raw[b][h][i] * scale;
                        const _Float16 hi = (_Float16) f;
                        v[i] = lowpart ? (_Float16) (f - (float) hi) : hi;
                    }
                }
                xb[b][h] = v;
                asm volatile("" : "+v"(xb[b][h]));   // consumed here: no ordinary load of the inputs is in flight once the tiles are requested
            }
    }
    const u32 tiles = (rows + 15) / 16;
    const u32 lds0 = __builtin_amdgcn_readfirstlane(lds_offset(tile0)), lds1 = lds0 + 16 * pitch;
    // the load instructions a tile costs this wave: its rows (w, w + W, .. < 16) times the 1 KiB pieces of a row
    const u32 mine = ((16 - wave + W - 1) / W) * ((rb / 16 + 63) / 64);
    float bv = -__builtin_inff();
    u32 bi = 0xffffffffu;
    u32 t = blockIdx.x, it = 0;
    if (t < tiles) head_tile_issue<W>(w, rows, rb, t, lds0, wave, lane);
    for (; t < tiles; t += gridDim.x, it++) {
        const u32 tn = t + gridDim.x;
        if (tn < tiles) head_tile_issue<W>(w, rows, rb, tn, (it & 1) ? lds0 : lds1, wave, lane);
        // this tile's requests of this wave have landed; the next tile's (the youngest in the queue) may stay in flight -
        // unless logits are stored in the loop: a store is not ordered with the loads
        if (tn < tiles && !logits) {
            if (mine >= 12) wait_vm<12>();
            else if (mine >= 10) wait_vm<10>();
            else if (mine >= 8) wait_vm<8>();
            else if (mine >= 4) wait_vm<4>();
            else wait_vm<0>();
        } else {
            wait_vm<0>();
        }
        __syncthreads();                                  // ... and every other wave's
        const u8* tb = tile0 + (it & 1) * 16 * pitch;
        const u8* arow = tb + n16 * pitch + wave * nbw * 34;      // A: row n16 of the tile, the wave's share of k
        const u8* drow = tb + (4 * g4) * pitch + wave * nbw * 34;  // scales: rows 4 g4 + r
        float tot[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int b = 0; b < NBM; b++) {
            if (FULL || (u32) b < nbw) {
                const u8* ab = arow + b * 34 + 2 + 4 * g4;
                const u32 q0 = *(const u16*) ab | ((u32) *(const u16*) (ab + 2) << 16);
                const u32 q1 = *(const u16*) (ab + 16) | ((u32) *(const u16*) (ab + 18) << 16);
                f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(head_codes_f16(q0), xb[b][0], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(head_codes_f16(q1), xb[b][1], acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const _Float16 d = __builtin_bit_cast(_Float16, *(const u16*) (drow + r * pitch + b * 34));
                    tot[r] = __builtin_fmaf((float) d, acc[r], tot[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) red[wave][(4 * g4 + r) * 16 + n16] = tot[r];
        __syncthreads();
        if (tid < 256) {
            // thread (row = tid / 16, n = tid % 16): the waves' sums in wave order, then high part + low part
            float s = red[0][tid];
#pragma unroll
            for (int v = 1; v < W; v++) s += red[v][tid];
            const float o = lane_xor<1>(s, lane);
            const u32 n = tid & 15, j = n >> 1, row = 16 * t + (tid >> 4);
            if ((n & 1) == 0 && j < m && row < rows) {
                float v = (s + o) * s_inv[j];
                if (logits) logits[(u64) j * ls + row] = v;
                if (v != v) v = -__builtin_inff();
                argmax_merge(bv, bi, v, row);
            }
        }
    }
    // the workgroup's best row per input: thread (row slot tid / 16, n) holds the best of its row slot
    if (tid < 256) {
        s_bv[tid] = bv;
        s_bi[tid] = bi;
    }
    __syncthreads();
    if (tid < 8) {
        float v = -__builtin_inff();
        u32 i = 0xffffffffu;
        for (u32 r = 0; r < 16; r++) argmax_merge(v, i, s_bv[r * 16 + 2 * tid], s_bi[r * 16 + 2 * tid]);
        part[((u64) blockIdx.x * 8 + tid) * 2] = f32_bits(v);
        part[((u64) blockIdx.x * 8 + tid) * 2 + 1] = i;
    }
}

extern "C" __global__ void __launch_bounds__(256, 2) head_q8_0_argmax_mfma(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part,
                                                                           u32 rows, u32 cols, u32 m) {
    head_mfma_body<4>(w, x, xs, logits, ls, part, rows, cols, m);
}
// The same for rows of up to 3072 columns (6 waves, block 384) and up to 4096 (8 waves, block 512): a wave still owns at
// most 512 columns, the tiles take all of a CU's LDS but for a workgroup's share, so one workgroup a CU.
// Rows of exactly 2048 columns on 8 waves: the same LDS a workgroup, twice the waves a SIMD to cover the tile reads' latency.
extern "C" __global__ void __launch_bounds__(512, 2) head_q8_0_argmax_mfma_n8(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part,
                                                                              u32 rows, u32 cols, u32 m) {
    head_mfma_body<8, 2048, true>(w, x, xs, logits, ls, part, rows, cols, m);
}
extern "C" __global__ void __launch_bounds__(384) head_q8_0_argmax_mfma_w6(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part,
                                                                           u32 rows, u32 cols, u32 m) {
    head_mfma_body<6>(w, x, xs, logits, ls, part, rows, cols, m);
}
extern "C" __global__ void __launch_bounds__(512) head_q8_0_argmax_mfma_w8(const u8* w, const float* x, u32 xs, float* logits, u32 ls, u32* part,
                                                                           u32 rows, u32 cols, u32 m) {
    head_mfma_body<8>(w, x, xs, logits, ls, part, rows, cols, m);
}

// part[(p * ts + j) * 2], + 1 = the largest of slice p (4096 values) of row j of logits (rows ls apart, n values a row) and its
// index, ties to the lower index: the first step of the arg-max for a head whose product kernel has none fused in (any type
// matvec_cols takes; the reference's mv_cols + topk_rows_at, session.rs:7034-7052).  grid = (ceil(n / 4096), m), block 256.
extern "C" __global__ void __launch_bounds__(256) argmax_slices(const float* logits, u32 ls, u32 n, u32* part, u32 ts) {
    __shared__ float sv[256];
    __shared__ u32 si[256];
    const u32 p = blockIdx.x, j = blockIdx.y, tid = threadIdx.x;
    const float* row = logits + (u64) j * ls;
    float bv = -__builtin_inff();
    u32 bi = 0xffffffffu;
#pragma unroll 4
    for (u32 q = 0; q < 16; q++) {
        const u32 i = p * 4096 + q * 256 + tid;
        if (i < n) argmax_merge(bv, bi, row[i], i);
    }
    sv[tid] = bv;
    si[tid] = bi;
    __syncthreads();
    for (u32 s = 128; s > 0; s >>= 1) {
        if (tid < s) {
            float v = sv[tid];
            u32 i = si[tid];
            argmax_merge(v, i, sv[tid + s], si[tid + s]);
            sv[tid] = v;
            si[tid] = i;
        }
        __syncthreads();
    }
    if (tid == 0) {
        part[((u64) p * ts + j) * 2] = f32_bits(sv[0]);
        part[((u64) p * ts + j) * 2 + 1] = si[0];
    }
}

// argmax_merge_parts for all m <= 8 rows and the greedy acceptance in one launch (the end of a verify round: one launch and
// its boundary less): ids[j] as there, then out[0] = keep = 1 + the number of leading drafts d[i] that equal ids[i], out[1] =
// the bonus token ids[keep - 1] (verify_accept in kernels/moe.hip; engine.rs:2377-2408).  grid 1, block 1024 (128 threads a row).
extern "C" __global__ void __launch_bounds__(1024) argmax_merge_accept(const u32* part, u32 nparts, u32 ts, u32* ids, u32 m, const u32* drafts,
                                                                       u32 n_drafts, u32* out) {
    __shared__ float sv[8][128];
    __shared__ u32 si[8][128];
    const u32 j = threadIdx.x >> 7, t = threadIdx.x & 127;
    float bv = -__builtin_inff();
    u32 bi = 0xffffffffu;
    if (j < m)
        for (u32 p = t; p < nparts; p += 128) argmax_merge(bv, bi, bits_f32(part[((u64) p * ts + j) * 2]), part[((u64) p * ts + j) * 2 + 1]);
    sv[j][t] = bv;
    si[j][t] = bi;
    __syncthreads();
    for (u32 s = 64; s > 0; s >>= 1) {
        if (t < s) {
            float v = sv[j][t];
            u32 i = si[j][t];
            argmax_merge(v, i, sv[j][t + s], si[j][t + s]);
            sv[j][t] = v;
            si[j][t] = i;
        }
        __syncthreads();
    }
    if (threadIdx.x < 64) {
        const u32 i = threadIdx.x;
        if (i < m) ids[i] = si[i][0];
        const u32 a = si[min(min(i, n_drafts), 7u)][0];
        const u32 d = i < n_drafts ? drafts[i] : 0u;
        const u64 stop = __builtin_amdgcn_ballot_w64(i >= n_drafts || a != d);
        const u32 first = (u32) __builtin_ctzll(stop);
        const u32 bonus = __builtin_amdgcn_readlane(a, first);
        if (i == 0) {
            out[0] = first + 1;
            out[1] = bonus;
        }
    }
}

// ids[j] = index of the largest of row j's `nparts` partial maxima part[(p * ts + j) * 2] (ties to the lower index).
// grid = m, block 256.
extern "C" __global__ void __launch_bounds__(256) argmax_merge_parts(const u32* part, u32 nparts, u32 ts, u32* ids, float* vals) {
    __shared__ float sv[256];
    __shared__ u32 si[256];
    const u32 j = blockIdx.x, tid = threadIdx.x;
    float bv = -__builtin_inff();
    u32 bi = 0xffffffffu;
    for (u32 p = tid; p < nparts; p += 256) {
        argmax_merge(bv, bi, bits_f32(part[((u64) p * ts + j) * 2]), part[((u64) p * ts + j) * 2 + 1]);
    }
    sv[tid] = bv;
    si[tid] = bi;
    __syncthreads();
    for (u32 s = 128; s > 0; s >>= 1) {
        if (tid < s) {
            float v = sv[tid];
            u32 i = si[tid];
            argmax_merge(v, i, sv[tid + s], si[tid + s]);
            sv[tid] = v;
            si[tid] = i;
        }
        __syncthreads();
    }
    if (tid == 0) {
        ids[j] = si[0];
        if (vals) vals[j] = sv[0];
    }
}
