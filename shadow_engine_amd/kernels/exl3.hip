// EXL3 (trellis-coded, Hadamard-rotated) matrix-vector products for 1..4 inputs, integer bit rates K = 1..8, codebook
// "mul1".  Format and arithmetic follow the CPU reference (crates/shadowzero-model/src/exl3.rs): a projection is a blob
// [suh f16[in] | svh f16[out] | 4-byte marker | trellis], the trellis is [in/16][out/16] tiles of 16 K u16 words, a tile is
// a ring of 256 K bits (most significant bit first inside little-endian u32 words) and weight t's 16-bit state ends at
// bit (t + 1) K; y = ((x * suh) H) W_hat H * svh with H the 128-point Walsh-Hadamard transform over 128-blocks.
//
// Lane map (wave64, made for this format rather than taken from the 32-lane tensor-core order the trellis was laid out
// for): one wave decodes the 8 tiles of one tile row of a 128-output block, which are 256 K contiguous bytes.  Lane
// L = 8 c + q takes weights 32 q .. 32 q + 31 of tile c: exactly K consecutive u32 words of the ring plus the word before
// them for the first windows, so every window position is a compile-time constant.  By the tile's position map
// (exl3.rs:106) those 32 weights are all 16 input rows of output columns q and q + 8 of the tile, so a lane owns two
// output columns outright and no cross-lane sum is needed inside a tile row.

__device__ __forceinline__ _Float16 exl3_cb2(u32 state) {
    // exl3.rs:87-94: the byte sum of state * 0x83DCD12D on top of 0x6400 is an f16 in [1024, 2048); one fused f16 multiply-add
    const u32 x = state * 0x83DCD12Du;
    const u32 s = __builtin_amdgcn_sad_u8(x, 0u, 0x6400u);
    const _Float16 h = __builtin_bit_cast(_Float16, (u16) s);
    return __builtin_fmaf16(h, __builtin_bit_cast(_Float16, (u16) 0x1eee), __builtin_bit_cast(_Float16, (u16) 0xc931));
}

// All 65,536 codebook values as f32 (crates/shadowzero-cuda/tests/exl3.rs:65-77 checks them bit for bit).
extern "C" __global__ void __launch_bounds__(256) exl3_codebook(float* out, u32 n) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (float) exl3_cb2(i);
}

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// state * 0x83DCD12D modulo 2^32: one v_mul_lo_u32, which issues at the full vector rate on this chip (measured: the same
// rate as the 24-bit multiply and the byte-sum instruction).
__device__ __forceinline__ u32 exl3_mul(u32 state) { return state * 0x83DCD12Du; }

// Two states to their two f16 weights at once: both byte sums land in one register as a pair of f16 bit patterns
// (v_sad_u8 into the low half, v_sad_hi_u8 into the high half, each on top of 0x6400), then one packed fused multiply-add.
// The same arithmetic per weight as exl3_cb2.
__device__ __forceinline__ f16x2 exl3_cb2_pair(u32 sa, u32 sb) {
    const u32 lo = __builtin_amdgcn_sad_u8(exl3_mul(sa), 0u, 0x64006400u);
    const u32 both = __builtin_amdgcn_sad_hi_u8(exl3_mul(sb), 0u, lo);
    const f16x2 h = __builtin_bit_cast(f16x2, both);
    const f16x2 kinv = {__builtin_bit_cast(_Float16, (u16) 0x1eee), __builtin_bit_cast(_Float16, (u16) 0x1eee)};
    const f16x2 kbias = {__builtin_bit_cast(_Float16, (u16) 0xc931), __builtin_bit_cast(_Float16, (u16) 0xc931)};
    return __builtin_elementwise_fma(h, kinv, kbias);
}

// Bit rates: K bits a weight, or K + 1/2 (H: positions alternate K and K + 1 bits, a pair takes 2 K + 1; exl3.rs:164).  A lane
// decodes 32 consecutive weights = EXL3_LANE_BITS stream bits; with a half rate that is an odd number of 16-bit halves, so
// every second lane of a tile starts in the middle of a word.
#define EXL3_LANE_BITS(K, H) (16 * (2 * (K) + (H)))          /* stream bits of a lane's 32 weights */
#define EXL3_TILE_WORDS(K, H) (4 * (2 * (K) + (H)))          /* u32 words of a tile's ring: 8 K, or 4 (2 K + 1) */
#define EXL3_NW(K, H) ((K) + 1 + (H))                        /* words S[] of a lane: the 32 stream bits before its own, then its own */

// End of the window of the lane's weight i, in stream bits after the lane's first own bit (Rate::end_bit, exl3.rs:164).
template <int K, bool H>
__device__ __forceinline__ constexpr int exl3_end(int i) {
    return H ? (i >> 1) * (2 * K + 1) + ((i & 1) ? 2 * K + 1 : K) : (i + 1) * K;
}

// The state of the lane's weight i from S = the stream from 32 bits before the lane's own bits on (S[0] = the ring word
// before its own for an integer rate), and T = the same stream 16 bits on (T[n] = stream bits [32 n + 16, 32 n + 48)), so
// that every window lies inside one register.
template <int K, bool H = false>
__device__ __forceinline__ u32 exl3_state(const u32 (&S)[EXL3_NW(K, H)], const u32 (&T)[EXL3_NW(K, H) - 1], int i) {
    const int a = 16 + exl3_end<K, H>(i);   // first stream bit of the window, counted from the first bit of S[0]
    const int n = a / 32, r = a % 32;
    return r <= 16 ? __builtin_amdgcn_ubfe(S[n], 16 - r, 16) : __builtin_amdgcn_ubfe(T[n], 32 - r, 16);
}

// The 32 weights of a lane, as 16 pairs (weights 2 p and 2 p + 1).
template <int K, bool H = false>
__device__ __forceinline__ void exl3_decode32(const u32 (&S)[EXL3_NW(K, H)], f16x2 (&w)[16]) {
    u32 T[EXL3_NW(K, H) - 1];
#pragma unroll
    for (int n = 0; n < EXL3_NW(K, H) - 1; n++) T[n] = __builtin_amdgcn_alignbit(S[n], S[n + 1], 16);
#pragma unroll
    for (int p = 0; p < 16; p++) w[p] = exl3_cb2_pair(exl3_state<K, H>(S, T, 2 * p), exl3_state<K, H>(S, T, 2 * p + 1));
}

// Input row (0..15) and output-column half (0: column q, 1: column q + 8) of a lane's weight i.
#define EXL3_ROW(i) (2 * ((i) >> 3) + ((i) & 1) + 8 * (((i) >> 1) & 1))
#define EXL3_HALF(i) (((i) >> 2) & 1)

// The lane's words S[] of tile (kt, tile column 8 ob + c): `tr` is the trellis as u32 words, nt = out / 16.  Integer rate: the
// lane's own K words are one contiguous 4 K-byte load; the word before them wraps to the tile's last word for the first lane.
// Half rate: lane q's bits start q (16 K + 8) bits into the ring, in the middle of a word for odd q; it reads the words that
// hold the 32 bits before them and its own (cyclically) and, for odd q, shifts the lot by 16 bits.
template <int K, bool H = false>
__device__ __forceinline__ void exl3_load_words(const u32* __restrict__ tr, u32 nt, u32 kt, u32 ob, u32 lane, u32 (&S)[EXL3_NW(K, H)]) {
    const u32 c = lane >> 3, q = lane & 7;
    const u32* tile = tr + ((u64) kt * nt + ob * 8 + c) * EXL3_TILE_WORDS(K, H);
    if constexpr (H) {
        constexpr u32 RW = EXL3_TILE_WORDS(K, H), NW = EXL3_NW(K, H);
        const u32 odd = q & 1;
        const u32 first = q * EXL3_LANE_BITS(K, H) - 16 * odd;    // a multiple of 32: the word that holds the lane's first own bit
        const u32 w0 = first / 32 + RW - 1;                        // one word before it (cyclic)
        u32 L[NW + 1];
#pragma unroll
        for (u32 n = 0; n <= NW; n++) L[n] = tile[(w0 + n) % RW];
#pragma unroll
        for (u32 n = 0; n < NW; n++) S[n] = odd ? __builtin_amdgcn_alignbit(L[n], L[n + 1], 16) : L[n];
    } else {
        S[0] = tile[q == 0 ? 8 * K - 1 : q * K - 1];
        typedef u32 vec __attribute__((ext_vector_type(K), aligned(4)));
        if constexpr (K == 1) {
            S[1] = tile[q];
        } else {
            const vec v = *(const vec*) (tile + q * K);
#pragma unroll
            for (int d = 0; d < K; d++) S[d + 1] = v[d];
        }
    }
}

// W_hat[in][out] as f32, straight from the trellis (exl3.rs:242-256): the bit-exact decode hook.
// grid = (out / 128, in / 16), block 64.
template <int K, bool H = false>
__device__ __forceinline__ void exl3_decode_kernel(const u8* blob, float* what, u32 in_f, u32 out_f) {
    const u32 lane = threadIdx.x, ob = blockIdx.x, kt = blockIdx.y;
    const u32* tr = (const u32*) (blob + 2 * (u64) in_f + 2 * (u64) out_f + 4);
    u32 S[EXL3_NW(K, H)];
    exl3_load_words<K, H>(tr, out_f / 16, kt, ob, lane, S);
    f16x2 w[16];
    exl3_decode32<K, H>(S, w);
    const u32 col = ob * 128 + (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int i = 0; i < 32; i++) what[(u64) (kt * 16 + EXL3_ROW(i)) * out_f + col + 8 * EXL3_HALF(i)] = (float) w[i / 2][i % 2];
}

template <int h>
__device__ __forceinline__ void wht_stage(float& v0, float& v1, u32 lane) {
    const float p0 = lane_xor<h>(v0, lane), p1 = lane_xor<h>(v1, lane);
    // partner - own in the upper lane of a pair, own + partner in the lower: one multiply-add by -1 or +1 (exact)
    const float sgn = bits_f32(0x3f800000u | ((lane & h) ? 0x80000000u : 0u));
    v0 = __builtin_fmaf(v0, sgn, p0);
    v1 = __builtin_fmaf(v1, sgn, p1);
}

// 128-point Walsh-Hadamard transform inside one wave: the lane holds elements `lane` (v0) and `lane + 64` (v1).  Stages
// h = 1, 2, .. 32 cross lanes, h = 64 is the lane's own pair; then the 1/sqrt(128) factor (exl3.rs:583-599), which the
// raw form leaves out.
__device__ __forceinline__ void wht128_wave_raw(float& v0, float& v1, u32 lane) {
    wht_stage<1>(v0, v1, lane);
    wht_stage<2>(v0, v1, lane);
    wht_stage<4>(v0, v1, lane);
    wht_stage<8>(v0, v1, lane);
    wht_stage<16>(v0, v1, lane);
    wht_stage<32>(v0, v1, lane);
    const float a = v0 + v1, b = v0 - v1;
    v0 = a;
    v1 = b;
}

__device__ __forceinline__ void wht128_wave(float& v0, float& v1, u32 lane) {
    wht128_wave_raw(v0, v1, lane);
    v0 *= 0.08838835f;
    v1 *= 0.08838835f;
}

// The decode loop of one wave: the 8 tile rows of input block kb against the M rotated inputs in the wave's strip xw
// (input j at xw[j * 128 ..]); on return the strip holds the partial sums instead (column c of input j at xw[j * 128 + c]).
template <int K, int M, bool H = false>
__device__ __forceinline__ void exl3_wave_main(const u8* __restrict__ blob, u32 in_f, u32 out_f, u32 ob, u32 kb, float* xw, u32 lane) {
    const u32* tr = (const u32*) (blob + 2 * (u64) in_f + 2 * (u64) out_f + 4);
    const u32 nt = out_f / 16;
    u32 S[EXL3_NW(K, H)], Sn[EXL3_NW(K, H)];
    exl3_load_words<K, H>(tr, nt, kb * 8, ob, lane, S);
    float acc[2][M];
#pragma unroll
    for (int j = 0; j < M; j++) acc[0][j] = acc[1][j] = 0.0f;
#pragma unroll 1
    for (u32 t = 0; t < 8; t++) {
        if (t < 7) exl3_load_words<K, H>(tr, nt, kb * 8 + t + 1, ob, lane, Sn);   // the next tile row's words, in flight while this one decodes
        f16x2 w[16];
        exl3_decode32<K, H>(S, w);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            // weights 8 q .. 8 q + 7 sit on input rows 2 q, 2 q + 1, 2 q + 8, 2 q + 9 of the tile row
            float xa[M][4];
#pragma unroll
            for (int j = 0; j < M; j++) {
                const float* xr = xw + j * 128 + t * 16 + 2 * q;
                xa[j][0] = xr[0];
                xa[j][1] = xr[1];
                xa[j][2] = xr[8];
                xa[j][3] = xr[9];
            }
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int i = 8 * q + e;
                const int r = (e & 1) + 2 * ((e >> 1) & 1);
#pragma unroll
                for (int j = 0; j < M; j++) acc[EXL3_HALF(i)][j] = __builtin_fmaf((float) w[i / 2][i % 2], xa[j][r], acc[EXL3_HALF(i)][j]);
            }
        }
#pragma unroll
        for (int d = 0; d < EXL3_NW(K, H); d++) S[d] = Sn[d];
    }
    __builtin_amdgcn_wave_barrier();
    const u32 col = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int j = 0; j < M; j++) {
        xw[j * 128 + col] = acc[0][j];
        xw[j * 128 + col + 8] = acc[1][j];
    }
}

// One wave = one 128-block of inputs (8 tile rows) of one 128-output block of one group: it rotates its block of every
// input (x * suh, then the transform) into a wave-private strip of LDS, decodes its 8 x 8 tiles into the partial sums of
// (x * suh) H W_hat for its two output columns a lane, and leaves them in its strip for the workgroup to add up.
template <int K, int M, bool H = false>
__device__ __forceinline__ void exl3_wave_body(const u8* __restrict__ blob, const float* __restrict__ x, u32 xs, const u32* __restrict__ rec,
                                               u32 n, u32 in_f, u32 out_f, u32 ob, u32 kb, float* xw, u32 lane) {
    const u16* suh = (const u16*) blob;
    const float s0 = f16_to_f32(suh[kb * 128 + lane]), s1 = f16_to_f32(suh[kb * 128 + 64 + lane]);
#pragma unroll
    for (int j = 0; j < M; j++) {
        float v0 = 0.0f, v1 = 0.0f;
        if ((u32) j < n) {
            const float* xj = x + (u64) rec[1 + j] * xs + kb * 128;
            v0 = xj[lane] * s0;
            v1 = xj[lane + 64] * s1;
            wht128_wave(v0, v1, lane);
        }
        xw[j * 128 + lane] = v0;
        xw[j * 128 + 64 + lane] = v1;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    exl3_wave_main<K, M, H>(blob, in_f, out_f, ob, kb, xw, lane);
}


// ------------------------------------------------------------------------------------- trellis rows through the LDS
// A wave's whole share of a projection (the 8 tile rows of its 128 x 128 block, 2 K KiB) is requested in one burst of
// global-to-LDS loads before it does anything else with the block: the loads need no registers, all of them are in
// flight while the wave rotates its input and decodes the first rows, and the decode loop stays rolled.  The loads are
// written as inline assembly on purpose: the compiler then keeps no count of them, so it does not hold back the first LDS
// read until every one of them has landed; exl3_rows_wait is the only thing that orders them.  Consequences for the
// caller: every ordinary global load whose value is still needed must have been consumed before exl3_rows_issue (a load
// the compiler waits for later would wait for the whole burst), and a wave must pass exl3_rows_wait<K>(7) before it ends.
// LDS layout of a tile row: decode lane L's K words start at word L * stride; K = 3 and 4 use the 16-byte lane pitch of
// the wide loads, the others are packed.  A wave's buffer is a ring of D rows (8, or fewer where more waves must fit a CU).  Rows are requested in units: one row by
// one load (K = 3, 4), two rows by one load (K = 2: a 512-byte row is half a load), one row by K one-word loads (the rest).
template <int K, int D = 8, bool H = false>
struct Exl3Rows {
    static_assert(D == 4 || D == 6 || D == 8, "ring depths in use");
    static constexpr int depth = D;                              // rows of the ring
    static constexpr int stride = (K == 3 || K == 4) ? 4 : K;
    static constexpr int src_words = 8 * EXL3_TILE_WORDS(K, H);  // words of a tile row of the block in memory
    // a half rate's row is copied as it lies, 64 words a load, the last load partly: 96, 160, 224 words in 128, 192, 256
    static constexpr int unit_rows = (!H && K == 2) ? 2 : 1;
    static constexpr int unit_loads = H ? (src_words + 63) / 64 : (K == 2 || K == 3 || K == 4) ? 1 : K;
    static constexpr int row_words = H ? 64 * unit_loads : 64 * stride;
    static constexpr int words = D * row_words;
    static constexpr int loads = D / unit_rows * unit_loads;   // of a full ring
    // loads that may still be in flight once the row t places behind the oldest requested one has landed
    static constexpr int after(int t) { return t >= D - 1 ? 0 : (D - 1 - t) / unit_rows * unit_loads; }
};

// Requests the unit that starts at row r (a multiple of unit_rows) of the wave's row stream into its ring slot r % D.
// row0 = the stream's first tile row (of the wave's 128-column block), pitch = words between tile rows, lds = the ring.
template <int K, int D = 8, bool H = false>
__device__ __forceinline__ void exl3_unit_issue(const u32* __restrict__ row0, u64 pitch, u32 r, u32 lane, u32 lds) {
    const u32 slot = r % D;
    if constexpr (H) {
        typedef Exl3Rows<K, D, H> R;
#pragma unroll
        for (int d = 0; d < R::unit_loads; d++)   // at least 32 lanes of every load are active: the wave always issues it
            if (d * 64 + lane < (u32) R::src_words) lds_load<4>(row0 + r * pitch + d * 64 + lane, lds + slot * 4 * R::row_words + d * 256);
    } else if constexpr (K == 4 || K == 3) {
        lds_load<4 * K>(row0 + r * pitch + lane * K, lds + slot * 1024);
    } else if constexpr (K == 2) {
        lds_load<16>(row0 + (r + (lane >> 5)) * pitch + (lane & 31) * 4, lds + slot * 512);   // lanes 0..31 row r, 32..63 row r + 1
    } else {
#pragma unroll
        for (int d = 0; d < K; d++) lds_load<4>(row0 + r * pitch + d * 64 + lane, lds + slot * 256 * K + d * 256);
    }
}

// The first D rows of a stream (every stream is a whole number of 8-row blocks).
template <int K, int D = 8, bool H = false>
__device__ __forceinline__ void exl3_rows_issue(const u32* __restrict__ row0, u64 pitch, u32 lane, u32 lds) {
#pragma unroll
    for (int r = 0; r < D; r += Exl3Rows<K, D, H>::unit_rows) exl3_unit_issue<K, D, H>(row0, pitch, r, lane, lds);
}

// Returns once the row t places behind the oldest request in flight has landed (with everything requested before it).
template <int K, int D = 8, bool H = false>
__device__ __forceinline__ void exl3_rows_wait(u32 t) {
    switch (t) {
        case 0: wait_vm<Exl3Rows<K, D, H>::after(0)>(); break;
        case 1: wait_vm<Exl3Rows<K, D, H>::after(1)>(); break;
        case 2: wait_vm<Exl3Rows<K, D, H>::after(2)>(); break;
        case 3: wait_vm<Exl3Rows<K, D, H>::after(3)>(); break;
        case 4: wait_vm<Exl3Rows<K, D, H>::after(4)>(); break;
        case 5: wait_vm<Exl3Rows<K, D, H>::after(5)>(); break;
        case 6: wait_vm<Exl3Rows<K, D, H>::after(6)>(); break;
        default: wait_vm<0>(); break;
    }
}

// The decode loop of one wave for one input over a stream of `rows` tile rows (8 a 128-block of inputs, consecutive
// blocks): the first D rows have been requested by exl3_rows_issue, every later row is requested into the ring slot of
// the row just decoded, so D rows stay in flight until the stream runs out.  xw holds the rotated input (16 values a
// row) and receives the wave's partial sums of its 128 output columns.
// XH: the wave's rotated inputs are f16 (exl3_put_x_f16: pairs of consecutive inputs a word, scaled by a power of two that
// `unscale` undoes) and two weights meet their two inputs in one v_dot2_f32_f16: 16 instructions a row for the products
// instead of 32, f32 sums as before, the inputs rounded to 11 bits.
template <int K, int D = 8, bool H = false, bool XH = false>
__device__ __forceinline__ void exl3_wave_stream(const u32* __restrict__ row0, u64 pitch, u32 rows, const u32* wb, u32 lds, float* xw, u32 lane,
                                                 float unscale = 1.0f) {
    typedef Exl3Rows<K, D, H> R;
    constexpr int stride = R::stride, ur = R::unit_rows;
    constexpr int NW = EXL3_NW(K, H);
    // where the lane's words lie in a row of the ring: an integer rate's K words at the lane's pitch and the word before them
    // (the tile's last for its first lane); a half rate's NW + 1 words around its bits, cyclic inside the tile (exl3_load_words)
    const u32 own = lane * stride, prev = ((lane & 7) == 0 ? lane + 7 : lane - 1) * stride + K - 1;
    u32 off[NW + 1];
    const u32 odd = lane & 1;
    if constexpr (H) {
        constexpr u32 RW = EXL3_TILE_WORDS(K, H);
        const u32 first = (lane & 7) * EXL3_LANE_BITS(K, H) - 16 * odd;
        const u32 w0 = first / 32 + RW - 1;
#pragma unroll
        for (int n = 0; n <= NW; n++) off[n] = (lane >> 3) * RW + (w0 + n) % RW;
    }
    float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll 1
    for (u32 r = 0; r < rows; r++) {
        exl3_rows_wait<K, D, H>(r + D > rows ? r + D - rows : 0);
        const u32* row = wb + (r & (D - 1)) * R::row_words;
        u32 S[NW];
        if constexpr (H) {
            u32 L[NW + 1];
#pragma unroll
            for (int n = 0; n <= NW; n++) L[n] = row[off[n]];
#pragma unroll
            for (int n = 0; n < NW; n++) S[n] = odd ? __builtin_amdgcn_alignbit(L[n], L[n + 1], 16) : L[n];
        } else {
            S[0] = row[prev];
#pragma unroll
            for (int d = 0; d < K; d++) S[d + 1] = row[own + d];
        }
        f16x2 w[16];
        exl3_decode32<K, H>(S, w);
        // once the row's words are in registers (the LDS reads have returned, not just been issued: a request that hits
        // in the cache can land within a few hundred cycles) its slot, with its partner's for two-row units, can take the
        // row D further on
        if ((r + 1) % ur == 0 && r + D + 1 - ur < rows) {
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
            exl3_unit_issue<K, D, H>(row0, pitch, r + D + 1 - ur, lane, lds);
        }
        if constexpr (XH) {
            // the row's 16 inputs as 8 f16 pairs: weights 2 j, 2 j + 1 of the lane meet inputs 2 q + {0, 1} (j even) or 2 q + 8 + {0, 1}
            // (j odd) of the tile row, q = j / 4
            typedef u32 u32x4v __attribute__((ext_vector_type(4)));
            const u32x4v lo = ((const u32x4v*) xw)[2 * r], hi = ((const u32x4v*) xw)[2 * r + 1];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const f16x2 xp = __builtin_bit_cast(f16x2, (j & 1) ? hi[j >> 2] : lo[j >> 2]);
                if ((j >> 1) & 1) acc1 = __builtin_amdgcn_fdot2(w[j], xp, acc1, false);
                else acc0 = __builtin_amdgcn_fdot2(w[j], xp, acc0, false);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float* xr = xw + r * 16 + 2 * q;
                const float xa[4] = {xr[0], xr[1], xr[8], xr[9]};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int i = 8 * q + e;
                    const int rr = (e & 1) + 2 * ((e >> 1) & 1);
                    if (EXL3_HALF(i)) acc1 = __builtin_fmaf((float) w[i / 2][i % 2], xa[rr], acc1);
                    else acc0 = __builtin_fmaf((float) w[i / 2][i % 2], xa[rr], acc0);
                }
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
    const u32 col = (lane >> 3) * 16 + (lane & 7);
    xw[col] = acc0 * unscale;
    xw[col + 8] = acc1 * unscale;
}

// A wave's rotated 128-block (the lane holds elements `lane` and `lane + 64`) as f16 in input order at xh[0..127], scaled by
// the power of two that takes the block's largest magnitude to [2^14, 2^15); returns what undoes the scale.
__device__ __forceinline__ float exl3_put_x_f16(u16* xh, float a0, float a1, u32 lane) {
    const float mx = wave_max_f32(fmaxf(__builtin_fabsf(a0), __builtin_fabsf(a1)));
    float scale, iv;
    pow2_scale_of(f32_bits(mx), scale, iv);
    xh[lane] = __builtin_bit_cast(u16, (_Float16) (a0 * scale));
    xh[lane + 64] = __builtin_bit_cast(u16, (_Float16) (a1 * scale));
    return iv;
}

// Group g = blockIdx.y: blob wtab[g], record gtab[17 g] = {n <= 4 (0: unused slot), xi[8], yi[8]}; wave w of the workgroup
// takes input block 4 blockIdx.z + w, and the four waves' sums are added in wave order into
// part[((g * gridDim.z + blockIdx.z) * 4 + j) * out + col], j < n.  grid = (out / 128, groups, ceil(in / 512)), block 256.
template <int K, bool H = false>
__device__ __forceinline__ void exl3_grouped_kernel(const u64* __restrict__ wtab, const u32* __restrict__ gtab, const float* __restrict__ x, u32 xs,
                                                    float* __restrict__ part, u32 in_f, u32 out_f) {
    __shared__ float xw_all[4][4 * 128];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // the wave index as a scalar: the index arithmetic on it is the scalar unit's
    const u32 kb = blockIdx.z * 4 + wave;
    const u32* rec = gtab + 17 * (u64) blockIdx.y;
    const u32 n = min(rec[0], 4u);
    if (n == 0) return;
    const u8* blob = (const u8*) wtab[blockIdx.y];
    float* xw = xw_all[wave];
    const bool live = kb < in_f / 128;
    if (live) {
        if (n == 1) exl3_wave_body<K, 1, H>(blob, x, xs, rec, n, in_f, out_f, blockIdx.x, kb, xw, lane);
        else if (n == 2) exl3_wave_body<K, 2, H>(blob, x, xs, rec, n, in_f, out_f, blockIdx.x, kb, xw, lane);
        else exl3_wave_body<K, 4, H>(blob, x, xs, rec, n, in_f, out_f, blockIdx.x, kb, xw, lane);
    }
    __syncthreads();
    const u32 nw = min(4u, in_f / 128 - blockIdx.z * 4);   // waves of this workgroup that had a block
    for (u32 p = threadIdx.x; p < n * 128; p += 256) {
        float v = xw_all[0][p];
        for (u32 w = 1; w < nw; w++) v += xw_all[w][p];
        part[(((u64) blockIdx.y * gridDim.z + blockIdx.z) * 4 + (p >> 7)) * out_f + blockIdx.x * 128 + (p & 127)] = v;
    }
}

#define EXL3_ENTRIES(K)                                                                                                              \
    extern "C" __global__ void __launch_bounds__(64) exl3_decode_##K(const u8* blob, float* what, u32 in_f, u32 out_f) {             \
        exl3_decode_kernel<K>(blob, what, in_f, out_f);                                                                              \
    }                                                                                                                                \
    extern "C" __global__ void __launch_bounds__(256) matvec_grouped_exl3_##K(const u64* wtab, const u32* gtab, const float* x, u32 xs, \
                                                                               float* part, u32 in_f, u32 out_f) {                     \
        exl3_grouped_kernel<K>(wtab, gtab, x, xs, part, in_f, out_f);                                                                \
    }

// K + 1/2 bits a weight (type ids 1030 + K, K = 1..3)
#define EXL3_HALF_ENTRIES(K)                                                                                                         \
    extern "C" __global__ void __launch_bounds__(64) exl3_decode_h##K(const u8* blob, float* what, u32 in_f, u32 out_f) {            \
        exl3_decode_kernel<K, true>(blob, what, in_f, out_f);                                                                        \
    }                                                                                                                                \
    extern "C" __global__ void __launch_bounds__(256) matvec_grouped_exl3h_##K(const u64* wtab, const u32* gtab, const float* x, u32 xs, \
                                                                                float* part, u32 in_f, u32 out_f) {                    \
        exl3_grouped_kernel<K, true>(wtab, gtab, x, xs, part, in_f, out_f);                                                          \
    }

EXL3_HALF_ENTRIES(1)
EXL3_HALF_ENTRIES(2)
EXL3_HALF_ENTRIES(3)

EXL3_ENTRIES(1)
EXL3_ENTRIES(2)
EXL3_ENTRIES(3)
EXL3_ENTRIES(4)
EXL3_ENTRIES(5)
EXL3_ENTRIES(6)
EXL3_ENTRIES(7)
EXL3_ENTRIES(8)

// The lane's two elements (`lane`, `lane + 64` of the 128-output block starting at `base`) of the sum over the zs partials
// of (group g, input j), in order.
__device__ __forceinline__ void exl3_part_sum2(const float* __restrict__ part, u32 g, u32 j, u32 zs, u32 out_f, u32 base, u32 lane, float& v0,
                                               float& v1) {
    v0 = 0.0f;
    v1 = 0.0f;
    for (u32 z = 0; z < zs; z++) {
        const float* p = part + (((u64) g * zs + z) * 4 + j) * out_f + base;
        v0 += p[lane];
        v1 += p[lane + 64];
    }
}

// y[yi[j]] = (sum of partials) H * svh for every input of every group: the output half of exl3.rs:557-564.
// grid = (out / 128, groups), block 64.
extern "C" __global__ void __launch_bounds__(64) exl3_finish_rows(const float* part, const u64* wtab, const u32* gtab, float* y, u32 ys,
                                                                  u32 in_f, u32 out_f) {
    const u32 lane = threadIdx.x, ob = blockIdx.x, g = blockIdx.y;
    const u32* rec = gtab + 17 * (u64) g;
    const u32 n = min(rec[0], 4u);
    if (n == 0) return;
    const u32 zs = (in_f / 128 + 3) / 4;
    const u16* svh = (const u16*) ((const u8*) wtab[g] + 2 * (u64) in_f) + ob * 128;
    const float s0 = f16_to_f32(svh[lane]), s1 = f16_to_f32(svh[lane + 64]);
    for (u32 j = 0; j < n; j++) {
        float v0, v1;
        exl3_part_sum2(part, g, j, zs, out_f, ob * 128, lane, v0, v1);
        wht128_wave(v0, v1, lane);
        float* o = y + (u64) rec[9 + j] * ys + ob * 128;
        o[lane] = v0 * s0;
        o[lane + 64] = v1 * s1;
    }
}

// ------------------------------------------------------------------------------------------- the fused verify layer
// A resident EXL3 layer for a verify batch (m <= 8 rows) in three launches, none of which needs a plan: the work items are
// the (token, expert) pairs themselves, one input each: pair p = j k + t of token j and rank t for p < m k, then the shared
// expert's pair m k + j of every token j.  Tokens that share an expert, and the shared expert for every token, read the
// same weights again; at 4 rows and top-10 of 512 that is about 10 % more reads, nearly all of them L2 hits, and it buys
// kernels with one input a wave: few registers, every wave of a launch resident at once.
// Expert e's three projections sit at ebase + e estride + {0, part, 2 part} (gate, up, down), the shared expert's at
// shbase + the same offsets (shbase = 0: no shared expert): addresses are computed, not looked up, so no load stands
// between a routing result and the first request for that expert's weights.
// pbuf holds u32 tidx[m k] | f32 w[m k] | u32 cnt[m].

// The rank-order sum of token j's finished down products for the 128 columns of block ob (launch 2 has finished every
// pair's block: no split over its inputs), column ob * 128 + tid for tid < 128: y[j] = sum over the cnt[j] experts of
// w[j, t] * dn[j k + t] + sigmoid(gl[j]) * dn[m k + j] (moe_combine_qwen_rows, kernels/forward.cu:2568).  Every load goes
// out before the first is waited for.  pbuf = u32 tidx[m k] | f32 w[m k] | u32 cnt[m].
__device__ __forceinline__ void exl3_combine_finished(const float* __restrict__ dn, const u8* __restrict__ pbuf, const float* __restrict__ gl,
                                                      float* __restrict__ y, u32 k, u32 m, u32 hidden, bool shared, u32 ob, u32 j, u32 tid) {
    const u32 G = m * k;
    const float* wts = (const float*) (pbuf + G * 4);
    const u32* cnt = (const u32*) (pbuf + 2 * G * 4);
    const u32 col = ob * 128 + tid;
    float v[17], w[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const u32 pair = j * k + min((u32) i, k - 1);
        v[i] = dn[(u64) pair * hidden + col];
        w[i] = wts[pair];
    }
    v[16] = shared ? dn[(u64) (G + j) * hidden + col] : 0.0f;
    const float sg = shared ? sigmoidf_ref(gl[j]) : 0.0f;
    const u32 c = cnt[j];
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++)
        if ((u32) i < c) a += w[i] * v[i];
    if (shared) a += sg * v[16];
    y[(u64) j * hidden + col] = a;
}

// The routing of a whole round in one launch, for a caller that has every layer's router logits before the first layer runs
// (sz_verify_round): wave (l, j) leaves token j's chosen experts, weights and count in layer l's plan, plans + l *
// plan_stride, in the layout above; launches 1 and 2 of those layers are then given no logits and read the plan instead of
// redoing the selection in every workgroup.  Same functions as the launches use, so the same bits.
// logits[l][m][ne]; grid = ceil(L m / 4), block 256; ne <= 512, k <= 16.
extern "C" __global__ void __launch_bounds__(256) verify_route_layers(const float* logits, u8* plans, u32 plan_stride, u32 ne, u32 k, u32 m, u32 L) {
    __shared__ double exs[4][512];
    __shared__ u32 tops[4][16];
    const u32 lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const u32 i = blockIdx.x * 4 + w;
    if (i >= L * m) return;
    const u32 l = i / m, j = i - l * m, G = m * k;
    const float* lg = logits + (u64) i * ne;
    u8* pbuf = plans + (u64) l * plan_stride;
    route_ids(lg, ne, k, lane, exs[w], tops[w]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    u32 kk;
    const float wt = route_weights(lg, ne, k, lane, tops[w], &kk);
    if (lane < k) {
        ((u32*) pbuf)[j * k + lane] = tops[w][lane];
        ((float*) (pbuf + G * 4))[j * k + lane] = wt;
    }
    if (lane == 0) ((u32*) (pbuf + 2 * G * 4))[j] = kk;
}

// Launch 1's workgroup: EXL3_GU_WAVES waves, each takes EXL3_VERIFY_NB consecutive 128-blocks of the input through a ring
// of EXL3_GU_DEPTH rows (grid z = ceil(hidden / 128 / (waves * blocks))).  One block a wave with a 4-row ring puts twice as
// many waves on a SIMD as two blocks a wave with an 8-row ring, for the same LDS: the waves spend most of their life
// waiting (for rows, for LDS, for an issue slot), and more of them hide more of it (24.2 -> 21.5 us a launch).  Four waves
// a workgroup rather than eight spread a little more evenly over the CUs (another 1 % of the round), at the price of twice
// the routing passes and partial sums.
#define EXL3_GU_WAVES 4
#define EXL3_VERIFY_NB 1
#define EXL3_GU_DEPTH 4

// Launch 1: routing (every workgroup of a routed pair redoes its token's selection on one of its waves; the workgroups
// with blockIdx.x == 0 and blockIdx.z == 0 of the gate half also publish tidx) and the gate and up products' partial
// sums: gup[((sel * S + pair) * zs + z)][ff], S = m (k + 1), sel 0 = gate, 1 = up, zs = gridDim.z.
// grid = (ff / 128, 2 S + c, zs), block 64 * EXL3_GU_WAVES; c = 0, or the rows that give (hidden / 128) m more workgroups
// for the sum of the layer before (cmode).
template <int K, bool H = false, bool XH = false>
__device__ __forceinline__ void verify_gate_up_kernel(const float* __restrict__ logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                      const float* __restrict__ u, u8* __restrict__ pbuf, float* __restrict__ gup, u32 ne, u32 k,
                                                      u32 m, u32 hidden, u32 ff, const float* __restrict__ cdn, const u8* __restrict__ cpbuf,
                                                      const float* __restrict__ cgl, float* __restrict__ cy, u32 cmode) {
    if (blockIdx.y >= 2 * (m * k + m)) {
        // rows of the grid past the pairs (cmode != 0): the rank-order sum of the layer before this one, whose launch 3 rides
        // here (same batch and shapes; cdn its finished down products, cpbuf its routing, cgl its shared gate logits, cy its
        // output; cmode 2: it has a shared expert), a workgroup a (token, 128-column block)
        const u32 ci = ((blockIdx.y - 2 * (m * k + m)) * gridDim.z + blockIdx.z) * gridDim.x + blockIdx.x, nb = hidden / 128;
        if (cmode && ci < nb * m && threadIdx.x < 128) exl3_combine_finished(cdn, cpbuf, cgl, cy, k, m, hidden, cmode == 2, ci % nb, ci / nb, threadIdx.x);
        return;
    }
    constexpr int NB = EXL3_VERIFY_NB, WA = EXL3_GU_WAVES, D = EXL3_GU_DEPTH;
    __shared__ __attribute__((aligned(16))) u32 wb_all[WA][Exl3Rows<K, D, H>::words];   // the waves' trellis rows; before that, the routing's scratch
    __shared__ float xw_all[WA][NB * 128];
    __shared__ u32 sc_all[WA][NB * 64];   // the wave's f16 input scales
    __shared__ u32 sv_out[64];            // the f16 output scales of the workgroup's 128 columns (wave 0 requests them)
    __shared__ u32 s_top[16];
    static_assert(sizeof(wb_all) >= 512 * sizeof(double), "the exact routing fallback needs 512 doubles");
    const u32 G = m * k, S = G + m;
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // the wave index as a scalar: the index arithmetic on it is the scalar unit's
    const u32 sel = blockIdx.y / S, pair = blockIdx.y % S;
    const u32 kbs = hidden / 128;
    const u32 kb0 = (blockIdx.z * WA + wave) * NB;
    const u32 nb = kb0 >= kbs ? 0u : min((u32) NB, kbs - kb0);   // this wave's input blocks: kb0 .. kb0 + nb - 1
    const u32 j = pair < G ? pair / k : pair - G;
    // the wave's blocks of its token's row do not depend on the routing: on their way while that is worked out
    float v[NB][2];
#pragma unroll
    for (int b = 0; b < NB; b++) {
        v[b][0] = v[b][1] = 0.0f;
        if ((u32) b < nb) {
            const float* xj = u + (u64) j * hidden + (kb0 + b) * 128;
            v[b][0] = load_f32_uncounted(xj + lane);      // waited for together with the input scales, behind which the trellis rows are already on their way
            v[b][1] = load_f32_uncounted(xj + lane + 64);
        }
    }
    u32* tidx = (u32*) pbuf;
    const u8* bp;
    if (pair < G && logits == nullptr) {
        // the round's routing launch has left every layer's chosen experts in its plan (verify_route_layers): one load
        const u32 e = tidx[pair];
        if (e == 0xffffffffu) return;
        bp = (const u8*) (ebase + e * estride + (u64) sel * part);
    } else if (pair < G) {
        const u32 t = pair % k;
        if (wave == (blockIdx.x + blockIdx.y + blockIdx.z) % WA) {   // not always the same wave: the prologues of co-resident workgroups spread over the SIMDs
            // the selection is a chain of dependent steps that the whole workgroup waits for: it goes ahead of the decoding
            // waves of other workgroups on its SIMD
            __builtin_amdgcn_s_setprio(3);
            route_id_of_rank(logits + (u64) j * ne, ne, k, t, lane, (double*) &wb_all[0][0], s_top);   // only s_top[t] is read
            __builtin_amdgcn_s_setprio(0);
            if (sel == 0 && blockIdx.x == 0 && blockIdx.z == 0 && lane == 0) tidx[pair] = s_top[t];
        }
        __syncthreads();
        const u32 e = s_top[t];
        if (e == 0xffffffffu) return;
        bp = (const u8*) (ebase + e * estride + (u64) sel * part);
    } else {
        if (!shbase) return;
        bp = (const u8*) (shbase + (u64) sel * part);
    }
    float* xw = xw_all[wave];
    if (nb) {
        const u32 sc_lds = __builtin_amdgcn_readfirstlane(lds_offset(sc_all[wave]));
        const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(wb_all[wave]));
        for (u32 b = 0; b < nb; b++) lds_load<4>(bp + (kb0 + b) * 256 + lane * 4, sc_lds + b * 256);
        if (wave == 0) lds_load<4>(bp + 2 * (u64) hidden + blockIdx.x * 256 + lane * 4, __builtin_amdgcn_readfirstlane(lds_offset(sv_out)));   // the block's output scales, for the end
        const u32* row0 = (const u32*) (bp + 2 * (u64) hidden + 2 * (u64) ff + 4) + ((u64) kb0 * 8 * (ff / 16) + blockIdx.x * 8) * EXL3_TILE_WORDS(K, H);
        const u64 pitch = (u64) (ff / 16) * EXL3_TILE_WORDS(K, H);
        exl3_rows_issue<K, D, H>(row0, pitch, lane, wb_lds);
        wait_vm<Exl3Rows<K, D, H>::loads>();   // everything requested before the rows: the token's values, the scales
#pragma unroll
        for (int b = 0; b < NB; b++) {
            load_landed(v[b][0]);
            load_landed(v[b][1]);
        }
        const u16* sc = (const u16*) sc_all[wave];
        float unscale = 1.0f;
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if ((u32) b < nb) {
                float a0 = v[b][0] * f16_to_f32(sc[b * 128 + lane]), a1 = v[b][1] * f16_to_f32(sc[b * 128 + lane + 64]);
                wht128_wave(a0, a1, lane);
                if constexpr (XH) {
                    static_assert(!XH || NB == 1, "the f16 inputs of a wave are one 128-block");
                    unscale = exl3_put_x_f16((u16*) xw, a0, a1, lane);
                } else {
                    xw[b * 128 + lane] = a0;
                    xw[b * 128 + 64 + lane] = a1;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        exl3_wave_stream<K, D, H, XH>(row0, pitch, 8 * nb, wb_all[wave], wb_lds, xw, lane, unscale);
    }
    __syncthreads();
    const u32 nw = min((u32) WA, (kbs - min(kbs, blockIdx.z * WA * NB) + NB - 1) / NB);   // waves of this workgroup that had blocks
    if (wave == 0) {
        // the workgroup's partial of its 128 columns, already through the output-side transform and the output scales (both
        // are linear, so launch 2 only has to add the zs partials up)
        float a0 = xw_all[0][lane], a1 = xw_all[0][lane + 64];
        for (u32 w = 1; w < nw; w++) {
            a0 += xw_all[w][lane];
            a1 += xw_all[w][lane + 64];
        }
        wht128_wave(a0, a1, lane);
        const u16* sv = (const u16*) sv_out;
        float* o = gup + ((u64) blockIdx.y * gridDim.z + blockIdx.z) * ff + blockIdx.x * 128;
        __builtin_nontemporal_store(a0 * f16_to_f32(sv[lane]), &o[lane]);
        __builtin_nontemporal_store(a1 * f16_to_f32(sv[lane + 64]), &o[lane + 64]);
    }
}

// Launch 2: act = silu(gate) * up of the pair, from the sums of launch 1's zs partials, by every wave for the 128-block of
// act it is about to use (16-fold redundant work of a hundred operations, instead of a launch), then the down
// product's partial sums: dn[pair * gridDim.z + z][hidden].  grid = (hidden / 128, S, ceil(ff / 512)), block 256.
template <int K, bool H = false, bool XH = false>
__device__ __forceinline__ void verify_down_kernel(const float* __restrict__ logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                   u8* __restrict__ pbuf, const float* __restrict__ gup, float* __restrict__ dn, u32 ne, u32 k, u32 m,
                                                   u32 hidden, u32 ff, u32 zs) {
    __shared__ __attribute__((aligned(16))) u32 wb_all[4][Exl3Rows<K, 8, H>::words];
    __shared__ float xw_all[4][128];
    __shared__ u32 sc_all[4][64];      // the wave's 128 f16 scales of down's inputs
    const u32 G = m * k, S = G + m;
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // the wave index as a scalar: the index arithmetic on it is the scalar unit's
    // Which (pair, column block) this workgroup takes.  Workgroup i of a launch runs on XCD i % 8, each with an L2 of its own,
    // and the 16 workgroups of a pair all read the pair's partial sums from launch 1: in launch order they sit on all eight
    // XCDs and the sums are fetched into eight L2s.  Where the shape allows, sets of 8 column blocks of one pair go to one
    // XCD instead (unit u = the set; the workgroups i with the same i % 8 and the same i / 64 share it), so two L2s fetch them.
    u32 pair = blockIdx.y, cbx = blockIdx.x;
    if (gridDim.z == 1 && gridDim.x % 8 == 0 && (gridDim.x / 8 * gridDim.y) % 8 == 0) {
        const u32 i = blockIdx.y * gridDim.x + blockIdx.x, unit = (i >> 6) * 8 + (i & 7), per = gridDim.x / 8;   // `per` runs a pair
        pair = unit / per;
        cbx = ((i >> 3) & 7) * per + unit % per;   // every per-th column block: the run's rows of the trellis spread over the row as the launch order's would
    }
    if (logits != nullptr && pair < G && pair % k == 0 && cbx == 0 && blockIdx.z == 0 && wave == 3) {
        // one wave a token: the routing weights and the count, for launch 3 (nothing in this launch reads them)
        const u32 j = pair / k;
        u32 kk;
        const float wt = route_weights(logits + (u64) j * ne, ne, k, lane, (const u32*) pbuf + pair, &kk);
        if (lane < k) ((float*) (pbuf + G * 4))[pair + lane] = wt;
        if (lane == 0) ((u32*) (pbuf + 2 * G * 4))[j] = kk;
    }
    const u32 kb = blockIdx.z * 4 + wave;
    const u32 kbs = ff / 128;
    // launch 1's partial sums of the wave's block of gate and up only depend on the pair: requested before its expert is known
    float g0 = 0.0f, g1 = 0.0f, u0 = 0.0f, u1 = 0.0f;
    float pv[4][4];
    u32 e = 0;
    if (pair < G) e = ((const u32*) pbuf)[pair];
    if (kb < kbs) {
        // the first four partials' loads all go out before any is waited for (a loop would take them a round trip at a time),
        // and without the compiler's count: the wave's rows are requested as soon as its expert is known, behind these loads
        // and without waiting for them, and the sums are taken once exactly these have landed
#pragma unroll
        for (int z = 0; z < 4; z++) {
            const u32 zz = min((u32) z, zs - 1);
            const float* pg = gup + ((u64) pair * zs + zz) * ff + kb * 128;
            const float* pu = gup + ((u64) (S + pair) * zs + zz) * ff + kb * 128;
            pv[z][0] = load_f32_uncounted(pg + lane);
            pv[z][1] = load_f32_uncounted(pg + lane + 64);
            pv[z][2] = load_f32_uncounted(pu + lane);
            pv[z][3] = load_f32_uncounted(pu + lane + 64);
        }
    }
    if (pair < G ? e == 0xffffffffu : shbase == 0) return;
    const u8* bp = (const u8*) (pair < G ? ebase + e * estride : shbase);
    float* xw = xw_all[wave];
    u32 svb0 = 0, svb1 = 0;   // wave 0 of a launch without a split over the inputs: down's output scales of the block (needed at the end)
    if (gridDim.z == 1 && wave == 0) {
        const u16* svh = (const u16*) (bp + 2 * (u64) part + 2 * (u64) ff) + cbx * 128;
        svb0 = load_u16_uncounted(svh + lane);
        svb1 = load_u16_uncounted(svh + lane + 64);
    }
    if (kb < kbs) {
        // no load the compiler counts is in flight here: what is, is counted by hand
        const u32 sc_lds = __builtin_amdgcn_readfirstlane(lds_offset(sc_all[wave]));
        const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(wb_all[wave]));
        const u8* down = bp + 2 * (u64) part;
        lds_load<4>(down + kb * 256 + lane * 4, sc_lds);                                  // down's input scales
        const u32* row0 = (const u32*) (down + 2 * (u64) ff + 2 * (u64) hidden + 4) + ((u64) kb * 8 * (hidden / 16) + cbx * 8) * EXL3_TILE_WORDS(K, H);
        const u64 pitch = (u64) (hidden / 16) * EXL3_TILE_WORDS(K, H);
        exl3_rows_issue<K, 8, H>(row0, pitch, lane, wb_lds);
        wait_vm<Exl3Rows<K, 8, H>::loads + 1>();   // the partial sums, requested before the burst, have landed
#pragma unroll
        for (int z = 0; z < 4; z++) {
#pragma unroll
            for (int c = 0; c < 4; c++) load_landed(pv[z][c]);
            if ((u32) z < zs) {
                g0 += pv[z][0];
                g1 += pv[z][1];
                u0 += pv[z][2];
                u1 += pv[z][3];
            }
        }
        for (u32 z = 4; z < zs; z++) {   // (hidden above 2048: these wait for the burst too)
            const float* pg = gup + ((u64) pair * zs + z) * ff + kb * 128;
            const float* pu = gup + ((u64) (S + pair) * zs + z) * ff + kb * 128;
            g0 += pg[lane];
            g1 += pg[lane + 64];
            u0 += pu[lane];
            u1 += pu[lane + 64];
        }
        // the wave's 128-block of act = silu(gate) * up (launch 1 left gate and up finished but for the sum over its
        // partials), rotated into the down projection's basis, into its strip
        wait_vm<Exl3Rows<K, 8, H>::loads>();
        const u16* suh = (const u16*) sc_all[wave];
        float a0 = (siluf_ref(g0) * u0) * f16_to_f32(suh[lane]);
        float a1 = (siluf_ref(g1) * u1) * f16_to_f32(suh[lane + 64]);
        wht128_wave(a0, a1, lane);
        float unscale = 1.0f;
        if constexpr (XH) {
            unscale = exl3_put_x_f16((u16*) xw, a0, a1, lane);
        } else {
            xw[lane] = a0;
            xw[64 + lane] = a1;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        exl3_wave_stream<K, 8, H, XH>(row0, pitch, 8, wb_all[wave], wb_lds, xw, lane, unscale);
    }
    __syncthreads();
    const u32 nw = min(4u, kbs - blockIdx.z * 4);
    if (gridDim.z == 1) {
        // the workgroup holds the whole sum over the inputs: it finishes its block here (output-side transform, scales), and
        // launch 3 only weights and adds
        if (wave == 0) {
            wait_vm<0>();
            load_landed(svb0);
            load_landed(svb1);
            const float sv0 = f16_to_f32((u16) svb0), sv1 = f16_to_f32((u16) svb1);
            float a0 = xw_all[0][lane], a1 = xw_all[0][lane + 64];
            for (u32 w = 1; w < nw; w++) {
                a0 += xw_all[w][lane];
                a1 += xw_all[w][lane + 64];
            }
            wht128_wave(a0, a1, lane);
            float* o = dn + (u64) pair * hidden + cbx * 128;
            __builtin_nontemporal_store(a0 * sv0, &o[lane]);
            __builtin_nontemporal_store(a1 * sv1, &o[lane + 64]);
        }
    } else if (threadIdx.x < 128) {
        float a = xw_all[0][threadIdx.x];
        for (u32 w = 1; w < nw; w++) a += xw_all[w][threadIdx.x];
        dn[((u64) pair * gridDim.z + blockIdx.z) * hidden + cbx * 128 + threadIdx.x] = a;
    }
}

// workgroups of 4 waves a CU that the LDS buffers leave room for (160 KiB a CU): the register budget follows it
#define EXL3_VERIFY_WAVES(K) ((K) <= 1 ? 8 : (K) == 2 ? 7 : (K) <= 4 ? 4 : (K) <= 5 ? 3 : 2)
// waves a SIMD of launch 1 that its LDS leaves room for (4-row rings)
#define EXL3_GU_OCC(K) ((K) <= 4 ? 8 : (K) == 5 ? 6 : 4)
#define EXL3_VERIFY_ENTRIES(K)                                                                                                            \
    extern "C" __global__ void __launch_bounds__(64 * EXL3_GU_WAVES, EXL3_GU_OCC(K)) verify_gate_up_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, \
                                                                                  const float* u, u8* pbuf, float* gup, u32 ne, u32 k, u32 m, \
                                                                                  u32 hidden, u32 ff, const float* cdn, const u8* cpbuf,      \
                                                                                  const float* cgl, float* cy, u32 cmode) {                   \
        verify_gate_up_kernel<K>(logits, ebase, estride, shbase, part, u, pbuf, gup, ne, k, m, hidden, ff, cdn, cpbuf, cgl, cy, cmode);   \
    }                                                                                                                                     \
    extern "C" __global__ void __launch_bounds__(256, EXL3_VERIFY_WAVES(K)) verify_down_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,   \
                                                                               u8* pbuf, const float* gup, float* dn, u32 ne, u32 k, u32 m,   \
                                                                               u32 hidden, u32 ff, u32 zs) {                                  \
        verify_down_kernel<K>(logits, ebase, estride, shbase, part, pbuf, gup, dn, ne, k, m, hidden, ff, zs);                             \
    }

// The same launches with the rotated inputs rounded to f16 and two products an instruction (session expert mode 3).
#define EXL3_VERIFY_F16_ENTRIES(K)                                                                                                        \
    extern "C" __global__ void __launch_bounds__(64 * EXL3_GU_WAVES, EXL3_GU_OCC(K)) verify_gate_up_exl3f_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, \
                                                                                  const float* u, u8* pbuf, float* gup, u32 ne, u32 k, u32 m, \
                                                                                  u32 hidden, u32 ff, const float* cdn, const u8* cpbuf,      \
                                                                                  const float* cgl, float* cy, u32 cmode) {                   \
        verify_gate_up_kernel<K, false, true>(logits, ebase, estride, shbase, part, u, pbuf, gup, ne, k, m, hidden, ff, cdn, cpbuf, cgl, cy, cmode); \
    }                                                                                                                                     \
    extern "C" __global__ void __launch_bounds__(256, EXL3_VERIFY_WAVES(K)) verify_down_exl3f_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part,   \
                                                                               u8* pbuf, const float* gup, float* dn, u32 ne, u32 k, u32 m,   \
                                                                               u32 hidden, u32 ff, u32 zs) {                                  \
        verify_down_kernel<K, false, true>(logits, ebase, estride, shbase, part, pbuf, gup, dn, ne, k, m, hidden, ff, zs);                \
    }

// K + 1/2 bits a weight: the LDS and register budget of the next whole rate
#define EXL3_VERIFY_HALF_ENTRIES(K)                                                                                                       \
    extern "C" __global__ void __launch_bounds__(64 * EXL3_GU_WAVES, EXL3_GU_OCC(K + 1)) verify_gate_up_exl3h_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, \
                                                                                  const float* u, u8* pbuf, float* gup, u32 ne, u32 k, u32 m, \
                                                                                  u32 hidden, u32 ff, const float* cdn, const u8* cpbuf,      \
                                                                                  const float* cgl, float* cy, u32 cmode) {                   \
        verify_gate_up_kernel<K, true>(logits, ebase, estride, shbase, part, u, pbuf, gup, ne, k, m, hidden, ff, cdn, cpbuf, cgl, cy, cmode); \
    }                                                                                                                                     \
    extern "C" __global__ void __launch_bounds__(256, EXL3_VERIFY_WAVES(K + 1)) verify_down_exl3h_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, \
                                                                               u8* pbuf, const float* gup, float* dn, u32 ne, u32 k, u32 m,   \
                                                                               u32 hidden, u32 ff, u32 zs) {                                  \
        verify_down_kernel<K, true>(logits, ebase, estride, shbase, part, pbuf, gup, dn, ne, k, m, hidden, ff, zs);                       \
    }

EXL3_VERIFY_HALF_ENTRIES(1)
EXL3_VERIFY_HALF_ENTRIES(2)
EXL3_VERIFY_HALF_ENTRIES(3)

EXL3_VERIFY_F16_ENTRIES(1)
EXL3_VERIFY_F16_ENTRIES(2)
EXL3_VERIFY_F16_ENTRIES(3)
EXL3_VERIFY_F16_ENTRIES(4)
EXL3_VERIFY_F16_ENTRIES(5)
EXL3_VERIFY_F16_ENTRIES(6)
EXL3_VERIFY_F16_ENTRIES(7)
EXL3_VERIFY_F16_ENTRIES(8)

EXL3_VERIFY_ENTRIES(1)
EXL3_VERIFY_ENTRIES(2)
EXL3_VERIFY_ENTRIES(3)
EXL3_VERIFY_ENTRIES(4)
EXL3_VERIFY_ENTRIES(5)
EXL3_VERIFY_ENTRIES(6)
EXL3_VERIFY_ENTRIES(7)
EXL3_VERIFY_ENTRIES(8)

// Launch 3: token j = blockIdx.y, output block blockIdx.x: y[j] = sum over its cnt[j] experts t, in rank order, of
// w[j,t] * (the finished down product of pair j k + t) + sigmoid(gl[j]) * (the shared expert's).  Wave t finishes expert t
// (wave k the shared one), then the first two waves add them up in rank order (moe_combine_qwen_rows,
// kernels/forward.cu:2568).  zs = launch 2's gridDim.z, or 0 when that was 1 and launch 2 has left finished blocks in dn:
// then 128 threads a workgroup do.  grid = (hidden / 128, m), block 1024 (k <= 16) or 128.
extern "C" __global__ void __launch_bounds__(1024) verify_combine_exl3(const float* dn, u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf,
                                                                       const float* gl, float* y, u32 k, u32 m, u32 hidden, u32 ff, u32 zs) {
    __shared__ float sums[17][128];
    const u32 lane = threadIdx.x & 63, t = threadIdx.x >> 6, ob = blockIdx.x, j = blockIdx.y;
    const u32 G = m * k;
    const u32* tidx = (const u32*) pbuf;
    const float* wts = (const float*) (pbuf + G * 4);
    const u32* cnt = (const u32*) (pbuf + 2 * G * 4);
    if (zs == 0) {
        if (t < 2) exl3_combine_finished(dn, pbuf, gl, y, k, m, hidden, shbase != 0, ob, j, threadIdx.x);
        return;
    }
    const u32 c = cnt[j];
    // one source's block: sum of its partials, output-side transform, scales, weight
    auto finish = [&](bool routed) {
        // everything that does not depend on the expert is requested first, all at once: the partial sums, the weight, the id
        const u32 pair = routed ? j * k + t : G + j;
        float v0 = 0.0f, v1 = 0.0f;
        for (u32 z = 0; z < zs; z++) {
            const float* p = dn + ((u64) pair * zs + z) * hidden + ob * 128;
            v0 += p[lane];
            v1 += p[lane + 64];
        }
        const u32 e = routed ? tidx[pair] : 0u;
        const float wt = routed ? wts[pair] : sigmoidf_ref(gl[j]);
        if (routed && t >= c) return;
        const u8* down = (const u8*) (routed ? ebase + e * estride : shbase) + 2 * (u64) part;
        const u16* svh = (const u16*) (down + 2 * (u64) ff) + ob * 128;
        const float s0 = f16_to_f32(svh[lane]), s1 = f16_to_f32(svh[lane + 64]);
        wht128_wave(v0, v1, lane);
        float* o = sums[routed ? t : 16];
        o[lane] = wt * (v0 * s0);
        o[lane + 64] = wt * (v1 * s1);
    };
    if (t < k) finish(true);
    if (shbase && t == (k < 16 ? k : 0)) finish(false);   // the shared expert on a wave of its own when there is one to spare
    __syncthreads();
    if (threadIdx.x < 128) {
        float a = 0.0f;
        for (u32 i = 0; i < c; i++) a += sums[i][threadIdx.x];
        if (shbase) a += sums[16][threadIdx.x];
        y[(u64) j * hidden + ob * 128 + threadIdx.x] = a;
    }
}

// ------------------------------------------------------------------------------------- the EXL3 head on the matrix cores
// The lm_head of an EXL3 checkpoint (in = hidden, out = vocabulary; kernels/exl3.cu:349-461, 610-625: exl3_rotate_rows_f32 and
// matvec_cols_exl3_pre of the reference) for the m <= 8 rows of a verify batch in one pass over the matrix, with the
// arg-max fused in.  The dot products run on the matrix cores (v_mfma_f32_16x16x16_f16, one a 16 x 16 tile): operand B is
// the tile, a lane supplying 4 CONSECUTIVE weights of the bit stream, which are input rows 2 a, 2 a + 1, 2 a + 8, 2 a + 9
// (a = lane / 16) of output column lane % 16 (exl3.rs:106); their four 16-bit windows lie in the 16 + 3 K stream bits
// that end at bit (t0 + 4) K, t0 = 32 (n % 8) + 8 a + 4 (n / 8): one funnel shift of two ring words (a per-lane constant
// choice) brings them into a register and the windows are then at fixed shifts (two shifts for K > 5).  Operand A is the
// input: row 2 j holds the f16 high part and row 2 j + 1 the f16 low part of token j's rotated input, scaled by the
// power of two that takes the token's largest rotated magnitude to [2^14, 2^15), in the same k order: every product with
// an f16 weight is exact, the matrix core adds in f32, and 8 tokens cost what one costs.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// Where element q (0..15) of a tile row's 16 inputs sits in the row's 16 slots of an A row: lane group a reads the slots
// 4 a .. 4 a + 3 = inputs 2 a, 2 a + 1, 2 a + 8, 2 a + 9 as one 8-byte word.
__device__ __forceinline__ u32 exl3_aslot(u32 q) { return 4 * ((q & 7) >> 1) + 2 * (q >> 3) + (q & 1); }

// Launch 1 of the head: token j = blockIdx.x.  Wave w rotates the 128-blocks w, w + waves, .. of x_j (x * suh, the
// transform), the largest magnitude over the row gives the token's scale, and the scaled values go out as f16 high and
// low parts: xa[(kb * 16 + 2 j + part) * 128 + 16 t8 + slot] for tile row t8 of block kb; inv[j] undoes the scale.
// grid = m, block = 64 * min(16, in / 128).
#define EXL3_HEAD_NB 4   /* 128-blocks a wave rotates at most: in <= 8192 */
extern "C" __global__ void __launch_bounds__(1024) exl3_head_rotate(const u8* blob, const float* x, u32 xs, u16* xa, float* inv, u32 in_f) {
    __shared__ float s_mx[16];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, nw = blockDim.x >> 6, j = blockIdx.x;
    const u32 kbs = in_f / 128;
    const u16* suh = (const u16*) blob;
    float rot[EXL3_HEAD_NB][2];
    float mx = 0.0f;
#pragma unroll
    for (int q = 0; q < EXL3_HEAD_NB; q++) {
        const u32 kb = wave + nw * q;
        rot[q][0] = rot[q][1] = 0.0f;
        if (kb < kbs) {
            const float* xj = x + (u64) j * xs + kb * 128;
            float a0 = xj[lane] * f16_to_f32(suh[kb * 128 + lane]), a1 = xj[lane + 64] * f16_to_f32(suh[kb * 128 + 64 + lane]);
            wht128_wave(a0, a1, lane);
            rot[q][0] = a0;
            rot[q][1] = a1;
            mx = fmaxf(mx, fmaxf(__builtin_fabsf(a0), __builtin_fabsf(a1)));
        }
    }
    mx = wave_max_f32(mx);
    if (lane == 0) s_mx[wave] = mx;
    __syncthreads();
    float all = 0.0f;
    for (u32 w = 0; w < nw; w++) all = fmaxf(all, s_mx[w]);
    float scale, iv;
    pow2_scale_of(f32_bits(all), scale, iv);
    if (threadIdx.x == 0) inv[j] = iv;
#pragma unroll
    for (int q = 0; q < EXL3_HEAD_NB; q++) {
        const u32 kb = wave + nw * q;
        if (kb < kbs) {
            u16* blk = xa + ((u64) kb * 16 + 2 * j) * 128;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const u32 i = lane + 64 * h;
                const float v = rot[q][h] * scale;
                const _Float16 hi = (_Float16) v;
                const _Float16 lo = (_Float16) (v - (float) hi);
                const u32 at = 16 * (i >> 4) + exl3_aslot(i & 15);
                blk[at] = __builtin_bit_cast(u16, hi);
                blk[128 + at] = __builtin_bit_cast(u16, lo);
            }
        }
    }
}

// Launch 2 of the head: output block ob = blockIdx.x (128 columns of the vocabulary).  Wave w of 4 takes the 128-blocks
// w, w + 4, .. of the input (8 tile rows each) through a ring of 4 rows; its A rows (2 m rows of 128 f16 a block, copied
// from xa once, in units of 4 rows) sit in LDS.  The four waves' sums are added in wave order, scaled back, taken through
// the output-side transform and scales, optionally stored as logits[j * ls + column], and the block's best column of every
// row goes to part[(ob * 8 + j) * 2] = {value bits, column} (a NaN counts as -inf, ties to the lower column).
// With a block list (sel[0] = n, sel[1 ..] = blocks; matvec_cols_exl3_pre_sparse of the reference, exl3.cu tail) workgroup
// i < n takes block sel[1 + i] and its logits and best go to place i instead of ob: logits[j * ls + 128 i + column in block];
// the arithmetic of a block does not depend on which workgroup runs it, so these are the bits the full pass gives.
// grid = out / 128 (or the list's bound), block 256, dynamic LDS = 4 * ceil(in / 512) * ceil(m / 2) KiB.
template <int K>
__device__ __forceinline__ void exl3_head_kernel(const u8* __restrict__ blob, const u16* __restrict__ xa, const float* __restrict__ inv,
                                                 float* __restrict__ logits, u32 ls, u32* __restrict__ part, u32 in_f, u32 out_f, u32 m,
                                                 const u32* __restrict__ sel) {
    constexpr int D = 4;
    typedef Exl3Rows<K, D> R;
    constexpr int stride = R::stride, ur = R::unit_rows;
    constexpr bool one_shift = 16 + 3 * K <= 32;
    extern __shared__ __attribute__((aligned(16))) u16 a_sh[];            // [wave][its blocks][4 nq A rows][128]; afterwards the waves' sums
    __shared__ __attribute__((aligned(16))) u32 wb_all[4][R::words];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, at = blockIdx.x;
    if (sel && at >= sel[0]) return;                                       // a list shorter than the grid
    const u32 ob = sel ? sel[1 + at] : at;
    const u32 kbs = in_f / 128, nkbw = (kbs + 3) / 4, nq = (m + 1) / 2;
    const u32 nkb = wave < kbs ? (kbs - wave + 3) / 4 : 0;                 // this wave's blocks: wave, wave + 4, ..
    const u32 nr = nkb * 8;
    const u32 nt = out_f / 16;
    const u64 pitch = (u64) nt * EXL3_TILE_WORDS(K, false);
    const u32* tr = (const u32*) (blob + 2 * (u64) in_f + 2 * (u64) out_f + 4) + (u64) ob * 8 * EXL3_TILE_WORDS(K, false);
    const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(wb_all[wave]));
    u16* aw = a_sh + (u64) wave * nkbw * nq * 512;                        // 512 f16 = 1 KiB = 4 A rows
    const u32 aw_lds = __builtin_amdgcn_readfirstlane(lds_offset(aw));
    // relative row i of the wave is tile row (wave + 4 (i / 8)) * 8 + i % 8 of the matrix
    auto row_ptr = [&](u32 i) -> const u32* { return tr + (u64) ((wave + 4 * (i >> 3)) * 8 + (i & 7)) * pitch; };
    auto issue = [&](u32 i) {                   // the unit that starts at relative row i (a multiple of ur) into its ring slot
        const u32 slot = i & (D - 1);
        if constexpr (K == 4 || K == 3) {
            lds_load<4 * K>(row_ptr(i) + lane * K, wb_lds + slot * 1024);
        } else if constexpr (K == 2) {
            lds_load<16>(row_ptr(i + (lane >> 5)) + (lane & 31) * 4, wb_lds + slot * 512);
        } else {
#pragma unroll
            for (int d = 0; d < K; d++) lds_load<4>(row_ptr(i) + d * 64 + lane, wb_lds + slot * 256 * K + d * 256);
        }
    };
    // the wave's A rows first (nq KiB a block), then its first rows
    for (u32 kbl = 0; kbl < nkb; kbl++)
        for (u32 qi = 0; qi < nq; qi++)
            lds_load<16>((const u8*) xa + ((u64) (wave + 4 * kbl) * 16 + 4 * qi) * 256 + lane * 16, aw_lds + (kbl * nq + qi) * 1024);
    u32 nring = 0;
    for (u32 i = 0; i < (u32) D && i < nr; i += ur) {
        issue(i);
        nring += R::unit_loads;
    }
    // the A rows have landed once only the ring's loads are in flight (at most 4 K of them: K <= 8)
    switch (nring) {
        case 0: wait_vm<0>(); break;
        case 1: wait_vm<1>(); break;
        case 2: wait_vm<2>(); break;
        case 3: wait_vm<3>(); break;
        case 4: wait_vm<4>(); break;
        case 5: wait_vm<5>(); break;
        case 6: wait_vm<6>(); break;
        case 7: wait_vm<7>(); break;
        case 8: wait_vm<8>(); break;
        case 12: wait_vm<12>(); break;
        case 16: wait_vm<16>(); break;
        case 20: wait_vm<20>(); break;
        case 24: wait_vm<24>(); break;
        case 28: wait_vm<28>(); break;
        case 32: wait_vm<32>(); break;
        default: wait_vm<0>(); break;
    }
    const u32 n = lane & 15, a = lane >> 4;
    const u32 t0 = 32 * (n & 7) + 8 * a + 4 * (n >> 3);
    // the 32 stream bits that end at bit e (exclusive) of the tile's ring: word jp holds the last of them, word jm the rest
    auto window = [&](u32 e, u32& om, u32& op, u32& sh) {
        const u32 jp = (e - 1) >> 5, jm = (jp + 8 * K - 1) % (8 * K);
        sh = 31 - ((e - 1) & 31);
        om = (jm / K) * stride + jm % K;   // a tile's word j sits at decode lane j / K, word j % K of that lane
        op = (jp / K) * stride + jp % K;
    };
    u32 om1, op1, sh1, om0 = 0, op0 = 0, sh0 = 0;
    window((t0 + 4) * K, om1, op1, sh1);
    if constexpr (!one_shift) window((t0 + 2) * K, om0, op0, sh0);
    f32x4 acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const bool fed = n < 2 * m;                            // this lane supplies A row n
    const u16* xa0 = aw + (fed ? n : 0) * 128 + 4 * a;
    const u32* wb = wb_all[wave];
    typedef u32 u32x2 __attribute__((ext_vector_type(2)));
    if constexpr (one_shift && ur == 1) {
        // Two tile rows a step on the 32-deep matrix instruction (a lane's 4 + 4 weights of the two rows' tiles against its 4 + 4
        // A values: the contraction runs over both rows' inputs), half the matrix instructions.  nr is a multiple of 8.
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
        typedef u32 u32x4v __attribute__((ext_vector_type(4)));
#pragma unroll 1
        for (u32 i = 0; i < nr; i += 2) {
            u32 w1[2][8][2];
            u32x2 xv[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const u32 r = i + h;
                exl3_rows_wait<K, D>(r + D > nr ? r + D - nr : 0);
                const u32* row = wb + (r & (D - 1)) * R::row_words;
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    w1[h][c][0] = row[c * 8 * stride + om1];
                    w1[h][c][1] = row[c * 8 * stride + op1];
                }
                xv[h] = *(const u32x2*) (xa0 + (u64) (r >> 3) * nq * 512 + 16 * (r & 7));
                if (!fed) xv[h] = u32x2{0u, 0u};
                if (r + D < nr) {
                    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the row's words are in registers, its slot can take the row D further on
                    issue(r + D);
                }
            }
            const f16x8 av = __builtin_bit_cast(f16x8, u32x4v{xv[0][0], xv[0][1], xv[1][0], xv[1][1]});
#pragma unroll
            for (int c = 0; c < 8; c++) {
                u32 b[2][2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const u32 hi = __builtin_amdgcn_alignbit(w1[h][c][0], w1[h][c][1], sh1);
                    const u32 s0 = __builtin_amdgcn_ubfe(hi, 3 * K, 16), s1 = __builtin_amdgcn_ubfe(hi, 2 * K, 16);
                    const u32 s2 = __builtin_amdgcn_ubfe(hi, K, 16), s3 = hi & 0xffffu;
                    b[h][0] = __builtin_bit_cast(u32, exl3_cb2_pair(s0, s1));
                    b[h][1] = __builtin_bit_cast(u32, exl3_cb2_pair(s2, s3));
                }
                const f16x8 bv = __builtin_bit_cast(f16x8, u32x4v{b[0][0], b[0][1], b[1][0], b[1][1]});
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc[c], 0, 0, 0);
            }
        }
    } else
#pragma unroll 1
    for (u32 i = 0; i < nr; i++) {
        exl3_rows_wait<K, D>(i + D > nr ? i + D - nr : 0);
        const u32* row = wb + (i & (D - 1)) * R::row_words;
        u32 w1[8][2], w0[8][2];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            w1[c][0] = row[c * 8 * stride + om1];
            w1[c][1] = row[c * 8 * stride + op1];
            if constexpr (!one_shift) {
                w0[c][0] = row[c * 8 * stride + om0];
                w0[c][1] = row[c * 8 * stride + op0];
            }
        }
        u32x2 xv = *(const u32x2*) (xa0 + (u64) (i >> 3) * nq * 512 + 16 * (i & 7));
        if (!fed) xv = u32x2{0u, 0u};
        // the row's words are in registers once the reads have returned: its slot can take the row D further on
        if ((i + 1) % ur == 0 && i + D + 1 - ur < nr) {
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
            issue(i + D + 1 - ur);
        }
        const f16x4 av = __builtin_bit_cast(f16x4, xv);
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const u32 hi = __builtin_amdgcn_alignbit(w1[c][0], w1[c][1], sh1);
            u32 s0, s1;
            if constexpr (one_shift) {
                s0 = __builtin_amdgcn_ubfe(hi, 3 * K, 16);
                s1 = __builtin_amdgcn_ubfe(hi, 2 * K, 16);
            } else {
                const u32 lo = __builtin_amdgcn_alignbit(w0[c][0], w0[c][1], sh0);
                s0 = __builtin_amdgcn_ubfe(lo, K, 16);
                s1 = lo & 0xffffu;
            }
            const u32 s2 = __builtin_amdgcn_ubfe(hi, K, 16), s3 = hi & 0xffffu;
            const f16x2 b01 = exl3_cb2_pair(s0, s1), b23 = exl3_cb2_pair(s2, s3);
            const f16x4 bv = {b01[0], b01[1], b23[0], b23[1]};
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x16f16(av, bv, acc[c], 0, 0, 0);
        }
    }
    __syncthreads();                                       // every wave is done with its A rows: the space takes the sums
    // D rows 4 a + i: lane group a holds tokens 2 a and 2 a + 1 (high part + low part each); red[wave][token][128]
    float* red = (float*) a_sh;
    {
        float* o = red + (u64) wave * m * 128;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            if (2 * a < m) o[(2 * a) * 128 + 16 * c + n] = acc[c][0] + acc[c][1];
            if (2 * a + 1 < m) o[(2 * a + 1) * 128 + 16 * c + n] = acc[c][2] + acc[c][3];
        }
    }
    __syncthreads();
    const u16* svh = (const u16*) (blob + 2 * (u64) in_f) + ob * 128;
    const float sv0 = f16_to_f32(svh[lane]), sv1 = f16_to_f32(svh[lane + 64]);
    for (u32 j = wave; j < m; j += 4) {
        float v0 = 0.0f, v1 = 0.0f;
        for (u32 w = 0; w < 4; w++) {
            v0 += red[((u64) w * m + j) * 128 + lane];
            v1 += red[((u64) w * m + j) * 128 + lane + 64];
        }
        const float iv = inv[j];
        v0 *= iv;
        v1 *= iv;
        wht128_wave(v0, v1, lane);
        v0 *= sv0;
        v1 *= sv1;
        const u32 c0 = ob * 128 + lane, c1 = c0 + 64;
        if (logits) {
            logits[(u64) j * ls + at * 128 + lane] = v0;
            logits[(u64) j * ls + at * 128 + lane + 64] = v1;
        }
        float bv = v0 != v0 ? -__builtin_inff() : v0;
        u32 bi = c0;
        argmax_merge(bv, bi, v1 != v1 ? -__builtin_inff() : v1, c1);
#pragma unroll
        for (int h = 1; h < 64; h <<= 1) {
            float ov;
            u32 oi;
            if (h == 1) { ov = lane_xor<1>(bv, lane); oi = f32_bits(lane_xor<1>(bits_f32(bi), lane)); }
            else if (h == 2) { ov = lane_xor<2>(bv, lane); oi = f32_bits(lane_xor<2>(bits_f32(bi), lane)); }
            else if (h == 4) { ov = lane_xor<4>(bv, lane); oi = f32_bits(lane_xor<4>(bits_f32(bi), lane)); }
            else if (h == 8) { ov = lane_xor<8>(bv, lane); oi = f32_bits(lane_xor<8>(bits_f32(bi), lane)); }
            else if (h == 16) { ov = lane_xor<16>(bv, lane); oi = f32_bits(lane_xor<16>(bits_f32(bi), lane)); }
            else { ov = lane_xor<32>(bv, lane); oi = f32_bits(lane_xor<32>(bits_f32(bi), lane)); }
            argmax_merge(bv, bi, ov, oi);
        }
        if (lane == 0) {
            part[((u64) at * 8 + j) * 2] = f32_bits(bv);
            part[((u64) at * 8 + j) * 2 + 1] = bi;
        }
    }
}

// ------------------------------------------------------------------------------------------ the 2-bit screen of the head
// An inexact, optional shortcut of the reference for the top-64 hand-off (exl3.cu:916-987, forward.cu:4371-4497,
// session.rs:5952-5995): a 2-bit copy of the head in the rotated basis scores every output cheaply, only the best 128-output
// blocks are then computed exactly.  Built once a head.  Block (ob, b) = outputs ob * 128 .., inputs b * 128 ..: the decoded
// weights of an input row are transformed over the block's 128 outputs (no 1/sqrt(128) here nor on the inputs: 1/128 once),
// times svh, rounded to f16; an output's 128 values of the block are then cut to the levels {-3, -1, 1, 3} * sh, sh = f16(0.5
// * 0.9957 * rms) (the optimal uniform four-level step of a Gaussian), the level u = 0..3 stored in two bits: the 16-byte
// group [(ob * 2 n_b + 2 b + hb) * 128 + r] holds inputs hb * 64 .. + 63 of output r, word wi bit 8 bi + 2 sl = input
// hb * 64 + 16 wi + 4 sl + bi (a byte lane a dot-product-of-four operand after a shift and a mask).  w_sc[(ob * n_b + b) * 128 + r] = sh.
// grid = (out / 128, in / 128), block 256.
template <int K>
__device__ __forceinline__ void exl3_q2_proxy_build(const u8* __restrict__ blob, u32* __restrict__ w_q2, u16* __restrict__ w_sc, u32 in_f, u32 out_f) {
    __shared__ _Float16 ws[4][16][130];       // a wave's tile row as decoded (f16 values): [input row][output]
    __shared__ u16 wh[128][130];              // the block in the rotated basis as f16: [output][input]
    const u32 wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ob = blockIdx.x, b = blockIdx.y;
    const u32 n_b = in_f / 128, nt = out_f / 16;
    const u32* tr = (const u32*) (blob + 2 * (u64) in_f + 2 * (u64) out_f + 4);
    const u16* svh = (const u16*) (blob + 2 * (u64) in_f) + ob * 128;
    const float sv0 = f16_to_f32(svh[lane]), sv1 = f16_to_f32(svh[lane + 64]);
    const u32 col = (lane >> 3) * 16 + (lane & 7);
    for (u32 kk = wave; kk < 8; kk += 4) {
        u32 S[EXL3_NW(K, false)];
        exl3_load_words<K>(tr, nt, b * 8 + kk, ob, lane, S);
        f16x2 w[16];
        exl3_decode32<K>(S, w);
#pragma unroll
        for (int i = 0; i < 32; i++) ws[wave][EXL3_ROW(i)][col + 8 * EXL3_HALF(i)] = w[i / 2][i % 2];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (u32 r = 0; r < 16; r++) {
            float v0 = (float) ws[wave][r][lane], v1 = (float) ws[wave][r][lane + 64];
            wht128_wave_raw(v0, v1, lane);
            // the product rounded to f32 first, then to f16, as the reference's two operations do: left to itself the compiler
            // makes one multiply-and-convert instruction of them, which rounds once and differs where the f32 product is an
            // f16 tie
            float p0 = v0 * 0.0078125f * sv0, p1 = v1 * 0.0078125f * sv1;
            asm volatile("" : "+v"(p0), "+v"(p1));
            wh[lane][kk * 16 + r] = __builtin_bit_cast(u16, (_Float16) p0);
            wh[lane + 64][kk * 16 + r] = __builtin_bit_cast(u16, (_Float16) p1);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    __syncthreads();
    if (threadIdx.x < 128) {
        const u32 r = threadIdx.x;
        float sq = 0.0f;
        for (u32 c = 0; c < 128; c++) {
            const float fv = f16_to_f32(wh[r][c]);
            sq = __builtin_fmaf(fv, fv, sq);
        }
        // the f32 square root correctly rounded, as the reference's sqrtf is: the f64 root of an f32 rounds to it (53 >= 2 * 24 + 2
        // bits); the single-precision instruction is an ulp off now and then
        const float delta = 0.9957f * (float) __builtin_sqrt((double) (sq * 0.0078125f));
        const u16 sh = __builtin_bit_cast(u16, (_Float16) (0.5f * delta));
        const float thr = 2.0f * f16_to_f32(sh);
        w_sc[((u64) ob * n_b + b) * 128 + r] = sh;
        for (u32 hb = 0; hb < 2; hb++) {
            u32x4 words;
#pragma unroll
            for (u32 wi = 0; wi < 4; wi++) {
                u32 pw = 0;
#pragma unroll
                for (u32 sl = 0; sl < 4; sl++)
#pragma unroll
                    for (u32 bi = 0; bi < 4; bi++) {
                        const float fv = f16_to_f32(wh[r][hb * 64 + wi * 16 + sl * 4 + bi]);
                        const u32 q = fv >= 0.0f ? (fv >= thr ? 3u : 2u) : (fv <= -thr ? 0u : 1u);
                        pw |= q << (bi * 8 + sl * 2);
                    }
                words[wi] = pw;
            }
            ((u32x4*) w_q2)[((u64) ob * (n_b * 2) + b * 2 + hb) * 128 + r] = words;
        }
    }
}

// The rows of a batch for the screen (exl3_rotate_rows_f32 + proxy_q2_quant_x of the reference: exl3.cu:610-625,
// forward.cu:4376-4420): block b of row j, (x * suh) transformed without the 1/sqrt(128) factor, as int8 codes with the
// scale amax / 127 (round half to even), four codes a word: xq[(j * n_b + b) * 32 + w] = inputs 4 w .. 4 w + 3 of the block;
// x_sc = the scale, x_corr = -3 * (sum of the codes) * scale (the levels are 2 u - 3 and the screen multiplies by u).
// grid = (in / 128, m), block 64.
extern "C" __global__ void __launch_bounds__(64) proxy_q2_quant_x(const u8* blob, const float* x, u32 xs, u32* xq, float* x_sc, float* x_corr, u32 in_f) {
    const u32 lane = threadIdx.x, b = blockIdx.x, j = blockIdx.y, n_b = in_f / 128;
    const u16* suh = (const u16*) blob + b * 128;
    const float* xj = x + (u64) j * xs + b * 128;
    float v0 = xj[lane] * f16_to_f32(suh[lane]), v1 = xj[lane + 64] * f16_to_f32(suh[lane + 64]);
    wht128_wave_raw(v0, v1, lane);
    const float amax = wave_max_f32(fmaxf(__builtin_fabsf(v0), __builtin_fabsf(v1)));
    const float sc = amax > 0.0f ? amax / 127.0f : 0.0f;
    const float inv = sc > 0.0f ? 1.0f / sc : 0.0f;
    const i32 q0 = (i32) __builtin_rintf(fmaxf(-127.0f, fminf(127.0f, v0 * inv)));
    const i32 q1 = (i32) __builtin_rintf(fmaxf(-127.0f, fminf(127.0f, v1 * inv)));
    u32 p0 = ((u32) q0 & 0xffu) << (8 * (lane & 3)), p1 = ((u32) q1 & 0xffu) << (8 * (lane & 3));
    p0 |= f32_bits(lane_xor<1>(bits_f32(p0), lane));
    p1 |= f32_bits(lane_xor<1>(bits_f32(p1), lane));
    p0 |= f32_bits(lane_xor<2>(bits_f32(p0), lane));
    p1 |= f32_bits(lane_xor<2>(bits_f32(p1), lane));
    u32* o = xq + ((u64) j * n_b + b) * 32;
    if ((lane & 3) == 0) {
        o[lane >> 2] = p0;
        o[16 + (lane >> 2)] = p1;
    }
    i32 tot = q0 + q1;
    tot += (i32) f32_bits(lane_xor<1>(bits_f32((u32) tot), lane));
    tot += (i32) f32_bits(lane_xor<2>(bits_f32((u32) tot), lane));
    tot += (i32) f32_bits(lane_xor<4>(bits_f32((u32) tot), lane));
    tot += (i32) f32_bits(lane_xor<8>(bits_f32((u32) tot), lane));
    tot += (i32) f32_bits(lane_xor<16>(bits_f32((u32) tot), lane));
    tot += (i32) f32_bits(lane_xor<32>(bits_f32((u32) tot), lane));
    if (lane == 0) {
        x_sc[(u64) j * n_b + b] = sc;
        x_corr[(u64) j * n_b + b] = -3.0f * (float) tot * sc;
    }
}

#define EXL3_HEAD_ENTRIES(K)                                                                                                          \
    extern "C" __global__ void __launch_bounds__(256) head_exl3_##K(const u8* blob, const u16* xa, const float* inv, float* logits, u32 ls, \
                                                                     u32* part, u32 in_f, u32 out_f, u32 m, const u32* sel) {             \
        exl3_head_kernel<K>(blob, xa, inv, logits, ls, part, in_f, out_f, m, sel);                                                    \
    }                                                                                                                                 \
    extern "C" __global__ void __launch_bounds__(256) exl3_build_q2_proxy_##K(const u8* blob, u32* w_q2, u16* w_sc, u32 in_f, u32 out_f) { \
        exl3_q2_proxy_build<K>(blob, w_q2, w_sc, in_f, out_f);                                                                        \
    }
EXL3_HEAD_ENTRIES(1)
EXL3_HEAD_ENTRIES(2)
EXL3_HEAD_ENTRIES(3)
EXL3_HEAD_ENTRIES(4)
EXL3_HEAD_ENTRIES(5)
EXL3_HEAD_ENTRIES(6)
EXL3_HEAD_ENTRIES(7)
EXL3_HEAD_ENTRIES(8)

// The one-matrix plan of a plain y_j = W x_j product for m <= 8 inputs: groups of 4 inputs, input row = output row = j.
// grid 1, block 64.
extern "C" __global__ void __launch_bounds__(64) cols_plan(u64* wtab, u32* gtab, u64 w, u32 m) {
    const u32 g = threadIdx.x;
    if (g * 4 >= m) return;
    wtab[g] = w;
    u32* r = gtab + 17 * g;
    r[0] = min(4u, m - 4 * g);
    for (u32 j = 0; j < 8; j++) {
        r[1 + j] = 4 * g + (j < 4 ? j : 0);
        r[9 + j] = 4 * g + (j < 4 ? j : 0);
    }
}

// --------------------------------------------------------------------------------- the verify layer on the matrix cores
// The same layer as verify_gate_up / verify_down above, for callers that accept f32 outputs within a tolerance instead of
// the exact per-weight arithmetic (the reference's mma_grouped_exl3_K beside its exact kernels, kernels/exl3.cu:682-725,
// held to 3e-3 of the largest output by crates/shadowzero-cuda/tests/exl3.rs:201).  Two things change.
// (1) The work items are the DISTINCT experts of the batch, not the (token, rank) pairs: a small first launch selects every
// token's experts and lists each expert once with the tokens that chose it, the shared expert as the first item with all of
// them, so an expert's weights are decoded once however many tokens use it.
// (2) The dot products run on the matrix cores, as in the head above: a lane decodes 4 consecutive weights of the bit stream,
// a 16 x 16 tile is one B operand of v_mfma_f32_16x16x16_f16, the item's tokens ride on the A rows as f16 high and low
// parts (8 tokens cost what one costs).  With LIN the codebook's last step is left to the end of the sum: a weight is
// f16(h k_inv + k_bias) with h = 1024 + the byte sum, an integer that IS an f16 as the byte-sum instruction leaves it, so
// the B operand is h itself and sum x w = k_inv sum x h + k_bias sum x, off from the exact value only by the rounding of
// each weight to f16 that is skipped (half a unit in the last place of a weight, about 1.5e-4 of an output, relative); the
// sum of a rotated block is sqrt(128) times the block's first element before the rotation.  Without LIN the weights are the
// codebook's bits and only the order of the f32 additions and the 22 bits kept of an input differ from the exact kernels.
// The plan: pbuf holds u32 tidx[m k] | f32 w[m k] | u32 cnt[m] as for the exact kernels, then at byte ioff (16-byte
// aligned) u32 n_items, 3 unused words, and 8 words an item: expert (0xffffffff: the shared one), n tokens, their rows as
// 8 bytes, their pair numbers as 8 u16 (pair j k + t of token j and rank t, m k + j for the shared expert: the row of the
// partial sums and of launch 2's output, which verify_combine_exl3 reads as it does after the exact launches).

// grid 1 (+ the workgroups of a riding sum), block 64 m.  Wave j selects token j's experts (lane t < k then holds rank t's); the items come out of three tables
// in LDS indexed by expert: the lowest pair that chose it (that pair's thread writes the item), the tokens that chose it as
// a bit mask, and each such token's rank.  The routing weights are not needed before launch 3 and are left to a spare
// workgroup of launch 1 (verify_route_weights below).
// Workgroups 1 .. (hidden / 128) m (cmode != 0): the rank-order sum of the layer before, as in verify_gate_up_kernel.
extern "C" __global__ void __launch_bounds__(512) verify_plan_exl3(const float* logits, u8* pbuf, u32 ioff, u32 ne, u32 k, u32 m, u32 shared, u32 hidden,
                                                                   const float* cdn, const u8* cpbuf, const float* cgl, float* cy, u32 cmode) {
    if (blockIdx.x > 0) {
        const u32 ci = blockIdx.x - 1, nb = hidden / 128;
        if (cmode && ci < nb * m)
            for (u32 t = threadIdx.x; t < 128; t += blockDim.x) exl3_combine_finished(cdn, cpbuf, cgl, cy, k, m, hidden, cmode == 2, ci % nb, ci / nb, t);
        return;
    }
    __shared__ double ex[8 * 512];   // the exact selection's scratch, a wave's 512 doubles
    __shared__ u32 top[8][16];
    __shared__ u32 lowest[512];      // expert -> the lowest pair number that chose it
    __shared__ u32 tokens[512];      // expert -> bit j: token j chose it
    __shared__ u8 rank[512 * 8];     // expert, token -> the token's rank of it
    __shared__ u32 wave_items[8];
    const u32 lane = threadIdx.x & 63, j = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), G = m * k;
    u32* tidx = (u32*) pbuf;
    u32* plan = (u32*) (pbuf + ioff);
    for (u32 i = threadIdx.x; i < 512; i += blockDim.x) {
        lowest[i] = 0xffffffffu;
        tokens[i] = 0;
    }
    route_ids(logits + (u64) j * ne, ne, k, lane, ex + j * 512, top[j]);
    __syncthreads();
    const u32 e = lane < k ? top[j][lane] : 0xffffffffu;
    const u32 p = j * k + lane;
    if (lane < k) tidx[p] = e;
    if (e != 0xffffffffu) {
        atomicMin(&lowest[e], p);
        atomicOr(&tokens[e], 1u << j);
        rank[e * 8 + j] = (u8) lane;
    }
    __syncthreads();
    const bool isf = e != 0xffffffffu && lowest[e] == p;
    const u64 firsts = __builtin_amdgcn_ballot_w64(isf);
    if (lane == 0) wave_items[j] = __builtin_popcountll(firsts);
    __syncthreads();
    u32 slot = shared ? 1u : 0u;
    for (u32 w = 0; w < j; w++) slot += wave_items[w];
    if (isf) {
        slot += __builtin_popcountll(firsts & ((1ull << lane) - 1));
        u32 n = 0;
        u64 toks = 0, pr0 = 0, pr1 = 0;
        for (u32 mask = tokens[e]; mask; mask &= mask - 1) {
            const u32 jj = __builtin_ctz(mask);
            toks |= (u64) jj << (8 * n);
            const u64 pv = jj * k + rank[e * 8 + jj];
            if (n < 4) pr0 |= pv << (16 * n);
            else pr1 |= pv << (16 * (n - 4));
            n++;
        }
        u32x4* rec = (u32x4*) (plan + 4 + 8 * slot);
        rec[0] = u32x4{e, n, (u32) toks, (u32) (toks >> 32)};
        rec[1] = u32x4{(u32) pr0, (u32) (pr0 >> 32), (u32) pr1, (u32) (pr1 >> 32)};
    }
    if (threadIdx.x == 0) {
        u32 count = shared ? 1u : 0u;
        for (u32 w = 0; w < m; w++) count += wave_items[w];
        plan[0] = count;
        if (shared) {
            u64 toks = 0, pr0 = 0, pr1 = 0;
            for (u32 jj = 0; jj < m; jj++) {
                toks |= (u64) jj << (8 * jj);
                const u64 pv = G + jj;
                if (jj < 4) pr0 |= pv << (16 * jj);
                else pr1 |= pv << (16 * (jj - 4));
            }
            u32x4* rec = (u32x4*) (plan + 4);
            rec[0] = u32x4{0xffffffffu, m, (u32) toks, (u32) (toks >> 32)};
            rec[1] = u32x4{(u32) pr0, (u32) (pr0 >> 32), (u32) pr1, (u32) (pr1 >> 32)};
        }
    }
}

// The renormalised routing weights and the counts of the chosen experts tidx (pbuf, as the plan left it) into w and cnt:
// a wave a token, for a workgroup that has nothing else to do.
__device__ __forceinline__ void verify_route_weights(const float* __restrict__ logits, u8* __restrict__ pbuf, u32 ne, u32 k, u32 m, u32 wave, u32 lane) {
    const u32 G = m * k;
    for (u32 j = wave; j < m; j += 4) {
        u32 kk;
        const float wt = route_weights(logits + (u64) j * ne, ne, k, lane, (const u32*) pbuf + j * k, &kk);
        if (lane < k) ((float*) (pbuf + G * 4))[j * k + lane] = wt;
        if (lane == 0) ((u32*) (pbuf + 2 * G * 4))[j] = kk;
    }
}

// Two states to the f16 pair (1024 + byte sum) that the codebook's multiply-add would start from.
__device__ __forceinline__ f16x2 exl3_h_pair(u32 sa, u32 sb) {
    const u32 lo = __builtin_amdgcn_sad_u8(exl3_mul(sa), 0u, 0x64006400u);
    return __builtin_bit_cast(f16x2, __builtin_amdgcn_sad_hi_u8(exl3_mul(sb), 0u, lo));
}

#define EXL3_KINV 0.0067672729f    /* f16 0x1eee */
#define EXL3_KBIAS (-10.3828125f)  /* f16 0xc931 */

// A wave's A rows in LDS: f16 astrip[(tile row * 2 NMAX + A row) * 16 + slot], A row 2 r the high and 2 r + 1 the low part
// of token r.  The lane holds elements `lane` (a0) and `lane + 64` (a1) of the token's rotated 128-block; they are scaled
// by the power of two that takes the block's largest magnitude to [2^14, 2^15) (returned inverse undoes it).
template <int NMAX>
__device__ __forceinline__ float exl3_put_a_rows(u16* astrip, u32 r, float a0, float a1, u32 lane) {
    const float mx = wave_max_f32(fmaxf(__builtin_fabsf(a0), __builtin_fabsf(a1)));
    float scale, iv;
    pow2_scale_of(f32_bits(mx), scale, iv);
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const u32 i = lane + 64 * h;
        const float v = (h ? a1 : a0) * scale;
        const _Float16 hi = (_Float16) v;
        const _Float16 lo = (_Float16) (v - (float) hi);
        u16* at = astrip + ((i >> 4) * (2 * NMAX) + 2 * r) * 16 + exl3_aslot(i & 15);
        at[0] = __builtin_bit_cast(u16, hi);
        at[16] = __builtin_bit_cast(u16, lo);
    }
    return iv;
}

// The decode loop of one wave on the matrix cores: the 8 tile rows of one 128-input block (requested into the ring by
// exl3_rows_issue) against the A rows in astrip; acc[c] = the 16 x 16 sums of column tile c (row 4 a + q of the lane group
// a = lane / 16: token 2 a high, low, token 2 a + 1 high, low; column lane % 16).
template <int K, bool LIN, int NMAX>
__device__ __forceinline__ void exl3_wave_mma(const u32* __restrict__ row0, u64 pitch, const u32* wb, u32 lds, const u16* astrip, u32 n, u32 lane,
                                              f32x4 (&acc)[8]) {
    constexpr int D = 4;
    typedef Exl3Rows<K, D> R;
    constexpr int stride = R::stride, ur = R::unit_rows;
    constexpr bool one_shift = 16 + 3 * K <= 32;
    const u32 n16 = lane & 15, a = lane >> 4;
    const u32 t0 = 32 * (n16 & 7) + 8 * a + 4 * (n16 >> 3);
    auto window = [&](u32 e, u32& om, u32& op, u32& sh) {
        const u32 jp = (e - 1) >> 5, jm = (jp + 8 * K - 1) % (8 * K);
        sh = 31 - ((e - 1) & 31);
        om = (jm / K) * stride + jm % K;
        op = (jp / K) * stride + jp % K;
    };
    u32 om1, op1, sh1, om0 = 0, op0 = 0, sh0 = 0;
    window((t0 + 4) * K, om1, op1, sh1);
    if constexpr (!one_shift) window((t0 + 2) * K, om0, op0, sh0);
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const bool fed = n16 < 2 * n;                          // this lane supplies A row n16
    const u16* xa0 = astrip + (fed ? n16 : 0) * 16 + 4 * a;
#pragma unroll 1
    for (u32 i = 0; i < 8; i++) {
        exl3_rows_wait<K, D>(i + D > 8 ? i + D - 8 : 0);
        const u32* row = wb + (i & (D - 1)) * R::row_words;
        u32 w1[8][2], w0[8][2];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            w1[c][0] = row[c * 8 * stride + om1];
            w1[c][1] = row[c * 8 * stride + op1];
            if constexpr (!one_shift) {
                w0[c][0] = row[c * 8 * stride + om0];
                w0[c][1] = row[c * 8 * stride + op0];
            }
        }
        typedef u32 u32x2 __attribute__((ext_vector_type(2)));
        u32x2 xv = *(const u32x2*) (xa0 + i * (2 * NMAX * 16));
        if (!fed) xv = u32x2{0u, 0u};
        if ((i + 1) % ur == 0 && i + D + 1 - ur < 8) {
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the row's words are in registers, its slot can take the row D further on
            exl3_unit_issue<K, D>(row0, pitch, i + D + 1 - ur, lane, lds);
        }
        const f16x4 av = __builtin_bit_cast(f16x4, xv);
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const u32 hi = __builtin_amdgcn_alignbit(w1[c][0], w1[c][1], sh1);
            u32 s0, s1;
            if constexpr (one_shift) {
                s0 = __builtin_amdgcn_ubfe(hi, 3 * K, 16);
                s1 = __builtin_amdgcn_ubfe(hi, 2 * K, 16);
            } else {
                const u32 lo = __builtin_amdgcn_alignbit(w0[c][0], w0[c][1], sh0);
                s0 = __builtin_amdgcn_ubfe(lo, K, 16);
                s1 = lo & 0xffffu;
            }
            const u32 s2 = __builtin_amdgcn_ubfe(hi, K, 16), s3 = hi & 0xffffu;
            const f16x2 b01 = LIN ? exl3_h_pair(s0, s1) : exl3_cb2_pair(s0, s1), b23 = LIN ? exl3_h_pair(s2, s3) : exl3_cb2_pair(s2, s3);
            const f16x4 bv = {b01[0], b01[1], b23[0], b23[1]};
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x16f16(av, bv, acc[c], 0, 0, 0);
        }
    }
}

// What a wave leaves for the workgroup's sum: red[(wave * NMAX + r) * 128 + column] = token r's partial sum of the wave's
// 128 inputs (high + low part, scale undone; with LIN times k_inv plus the token's k_bias term).  iv[h], cr[h]: the inverse
// scale and the k_bias term of the lane group's tokens 2 a + h.
template <bool LIN, int NMAX>
__device__ __forceinline__ void exl3_mma_to_red(float* red, u32 wave, u32 n, u32 lane, const f32x4 (&acc)[8], const float (&iv)[2], const float (&cr)[2]) {
    const u32 n16 = lane & 15, a = lane >> 4;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const u32 r = 2 * a + h;
        if (r < n && r < (u32) NMAX) {
            const float f = iv[h] * (LIN ? EXL3_KINV : 1.0f), c0 = LIN ? cr[h] : 0.0f;
            float* o = red + (wave * NMAX + r) * 128 + n16;
#pragma unroll
            for (int c = 0; c < 8; c++) o[16 * c] = __builtin_fmaf(acc[c][2 * h] + acc[c][2 * h + 1], f, c0);
        }
    }
}

// The LDS a workgroup of the two launches needs, in words, for ring rows of `ring` words a wave (Exl3Rows<K, 4>::words).
#define EXL3_MMA_WAVE_WORDS(ring, NMAX) ((ring) + (NMAX) * 128 + 64 + 16)   /* ring, A rows, input scales, the tokens' inverse scales and k_bias terms */
#define EXL3_MMA_LDS_WORDS(ring, NMAX) (4 * EXL3_MMA_WAVE_WORDS(ring, NMAX) + 64)

// Launch 1: the gate and up products of every item, partial sums gup[((sel * S + pair) * zs + z)][ff] as the exact launch
// leaves them (already through the output-side transform and scales).  grid = (ff / 128, 2 IT, zs), IT = the item slots
// (an even number above m k + 1), zs = ceil(hidden / 512); block 256; dynamic LDS EXL3_MMA_LDS_WORDS.
template <int K, bool LIN, int NMAX>
__device__ __forceinline__ void verify_gate_up_mma_kernel(const float* __restrict__ logits, u64 ebase, u64 estride, u64 shbase, u32 part,
                                                          const float* __restrict__ u, u8* __restrict__ pbuf, u32 ioff, float* __restrict__ gup, u32 ne,
                                                          u32 k, u32 m, u32 hidden, u32 ff) {
    constexpr int D = 4;
    typedef Exl3Rows<K, D> R;
    constexpr int WW = EXL3_MMA_WAVE_WORDS(R::words, NMAX);
    extern __shared__ __attribute__((aligned(16))) u32 dyn[];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32 IT = gridDim.y >> 1, sel = blockIdx.y >= IT ? 1u : 0u, it = blockIdx.y - sel * IT;
    const u32* plan = (const u32*) (pbuf + ioff);
    if (it >= plan[0]) {
        // the last item slot is never an item (there are at most m k + 1): one of its workgroups works the routing weights out
        // for launch 3 while the others multiply
        if (blockIdx.y == gridDim.y - 1 && blockIdx.x == 0 && blockIdx.z == 0) verify_route_weights(logits, pbuf, ne, k, m, wave, lane);
        return;
    }
    const u32* rec = plan + 4 + 8 * it;
    const u32 e = rec[0], n = min(rec[1], (u32) NMAX);
    const u64 toks = (u64) rec[2] | ((u64) rec[3] << 32);
    const u32 S = m * k + m;
    const u8* bp = (const u8*) (e == 0xffffffffu ? shbase : ebase + e * estride) + (u64) sel * part;
    const u32 kbs = hidden / 128, kb = blockIdx.z * 4 + wave;
    const bool live = kb < kbs;
    u32* wring = dyn + wave * WW;
    u16* astrip = (u16*) (wring + R::words);
    u32* sc = wring + R::words + NMAX * 128;
    u32* sv_out = dyn + 4 * WW;
    float iv[2] = {0.0f, 0.0f}, cr[2] = {0.0f, 0.0f};   // the inverse scales and the k_bias terms of the lane group's two tokens
    f32x4 acc[8];
    if (live) {
        float v[NMAX][2];
#pragma unroll
        for (int r = 0; r < NMAX; r++) {
            const u32 tok = (u32) (toks >> (8 * min((u32) r, n - 1))) & 0xffu;
            const float* xj = u + (u64) tok * hidden + kb * 128;
            v[r][0] = xj[lane];
            v[r][1] = xj[lane + 64];
        }
#pragma unroll
        for (int r = 0; r < NMAX; r++) asm volatile("" : "+v"(v[r][0]), "+v"(v[r][1]));   // no ordinary load is in flight from now on
        const u32 sc_lds = __builtin_amdgcn_readfirstlane(lds_offset(sc));
        const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(wring));
        lds_load<4>(bp + kb * 256 + lane * 4, sc_lds);
        if (wave == 0) lds_load<4>(bp + 2 * (u64) hidden + blockIdx.x * 256 + lane * 4, __builtin_amdgcn_readfirstlane(lds_offset(sv_out)));
        const u32* row0 = (const u32*) (bp + 2 * (u64) hidden + 2 * (u64) ff + 4) + ((u64) kb * 8 * (ff / 16) + blockIdx.x * 8) * EXL3_TILE_WORDS(K, false);
        const u64 pitch = (u64) (ff / 16) * EXL3_TILE_WORDS(K, false);
        exl3_rows_issue<K, D>(row0, pitch, lane, wb_lds);
        wait_vm<R::loads>();
        const u16* sch = (const u16*) sc;
        const float s0 = f16_to_f32(sch[lane]), s1 = f16_to_f32(sch[lane + 64]);
        // a token's inverse scale and k_bias term wait in LDS for the lanes that hold the token's sums at the end
        float* ivs = (float*) (sc + 64);
#pragma unroll
        for (int r = 0; r < NMAX; r++) {
            if ((u32) r < n) {
                float a0 = v[r][0] * s0, a1 = v[r][1] * s1;
                const float c0 = (EXL3_KBIAS * 11.3137085f) * bits_f32(__builtin_amdgcn_readlane(f32_bits(a0), 0));
                wht128_wave(a0, a1, lane);
                const float i0 = exl3_put_a_rows<NMAX>(astrip, r, a0, a1, lane);
                if (lane == 0) {
                    ivs[r] = i0;
                    ivs[NMAX + r] = c0;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        exl3_wave_mma<K, LIN, NMAX>(row0, pitch, wring, wb_lds, astrip, n, lane, acc);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const u32 r = min(2 * (lane >> 4) + h, (u32) NMAX - 1);
            iv[h] = ivs[r];
            cr[h] = ivs[NMAX + r];
        }
    }
    __syncthreads();   // every wave is done with its ring and A rows: the space takes the sums
    float* red = (float*) dyn;
    if (live) exl3_mma_to_red<LIN, NMAX>(red, wave, n, lane, acc, iv, cr);
    __syncthreads();
    const u32 nw = min(4u, kbs - blockIdx.z * 4);
    const u16* sv = (const u16*) sv_out;
    for (u32 r = wave; r < n; r += 4) {
        float a0 = 0.0f, a1 = 0.0f;
        for (u32 w = 0; w < nw; w++) {
            a0 += red[(w * NMAX + r) * 128 + lane];
            a1 += red[(w * NMAX + r) * 128 + lane + 64];
        }
        wht128_wave(a0, a1, lane);
        const u32 pair = (rec[4 + (r >> 1)] >> (16 * (r & 1))) & 0xffffu;
        float* o = gup + (((u64) sel * S + pair) * gridDim.z + blockIdx.z) * ff + blockIdx.x * 128;
        __builtin_nontemporal_store(a0 * f16_to_f32(sv[lane]), &o[lane]);
        __builtin_nontemporal_store(a1 * f16_to_f32(sv[lane + 64]), &o[lane + 64]);
    }
}

// Launch 2: act = silu(gate) * up of every token of the item from launch 1's partial sums (by every wave for its own
// 128-block, as the exact launch does), then the down product: finished blocks dn[pair][hidden] when one workgroup holds
// the whole sum over the inputs (ff <= 512), else partial sums dn[pair * gridDim.z + z][hidden] for verify_combine_exl3.
// grid = (hidden / 128, IT, ceil(ff / 512)), block 256, dynamic LDS as launch 1.
template <int K, bool LIN, int NMAX>
__device__ __forceinline__ void verify_down_mma_kernel(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* __restrict__ pbuf, u32 ioff,
                                                       const float* __restrict__ gup, float* __restrict__ dn, u32 k, u32 m, u32 hidden, u32 ff, u32 zs) {
    constexpr int D = 4;
    typedef Exl3Rows<K, D> R;
    constexpr int WW = EXL3_MMA_WAVE_WORDS(R::words, NMAX);
    extern __shared__ __attribute__((aligned(16))) u32 dyn[];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32 it = blockIdx.y;
    const u32* plan = (const u32*) (pbuf + ioff);
    if (it >= plan[0]) return;
    const u32* rec = plan + 4 + 8 * it;
    const u32 e = rec[0], n = min(rec[1], (u32) NMAX);
    const u32 S = m * k + m;
    const u8* down = (const u8*) (e == 0xffffffffu ? shbase : ebase + e * estride) + 2 * (u64) part;
    const u32 kbs = ff / 128, kb = blockIdx.z * 4 + wave;
    const bool live = kb < kbs;
    u32* wring = dyn + wave * WW;
    u16* astrip = (u16*) (wring + R::words);
    u32* sc = wring + R::words + NMAX * 128;
    u32* sv_out = dyn + 4 * WW;
    float iv[2] = {0.0f, 0.0f}, cr[2] = {0.0f, 0.0f};   // the inverse scales and the k_bias terms of the lane group's two tokens
    f32x4 acc[8];
    if (live) {
        // the sums of launch 1's partials of the wave's block of gate and up, every token's loads on their way at once (in
        // two lots of four tokens when there may be more)
        float gu[NMAX][4];
#pragma unroll
        for (int r0 = 0; r0 < NMAX; r0 += 4) {
            if (r0 > 0 && n <= (u32) r0) break;
            float pv[4][4][4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const u32 r = min((u32) (r0 + q), n - 1);
                const u32 pair = (rec[4 + (r >> 1)] >> (16 * (r & 1))) & 0xffffu;
#pragma unroll
                for (int z = 0; z < 4; z++) {
                    const u32 zz = min((u32) z, zs - 1);
                    const float* pg = gup + ((u64) pair * zs + zz) * ff + kb * 128;
                    const float* pu = gup + ((u64) (S + pair) * zs + zz) * ff + kb * 128;
                    pv[q][z][0] = pg[lane];
                    pv[q][z][1] = pg[lane + 64];
                    pv[q][z][2] = pu[lane];
                    pv[q][z][3] = pu[lane + 64];
                }
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    float t = pv[q][0][c];
#pragma unroll
                    for (int z = 1; z < 4; z++)
                        if ((u32) z < zs) t += pv[q][z][c];
                    gu[r0 + q][c] = t;
                }
                if (zs > 4) {
                    const u32 r = min((u32) (r0 + q), n - 1);
                    const u32 pair = (rec[4 + (r >> 1)] >> (16 * (r & 1))) & 0xffffu;
                    for (u32 z = 4; z < zs; z++) {
                        const float* pg = gup + ((u64) pair * zs + z) * ff + kb * 128;
                        const float* pu = gup + ((u64) (S + pair) * zs + z) * ff + kb * 128;
                        gu[r0 + q][0] += pg[lane];
                        gu[r0 + q][1] += pg[lane + 64];
                        gu[r0 + q][2] += pu[lane];
                        gu[r0 + q][3] += pu[lane + 64];
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < NMAX; r++) asm volatile("" : "+v"(gu[r][0]), "+v"(gu[r][1]), "+v"(gu[r][2]), "+v"(gu[r][3]));   // no ordinary load is in flight from now on
        const u32 sc_lds = __builtin_amdgcn_readfirstlane(lds_offset(sc));
        const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(wring));
        lds_load<4>(down + kb * 256 + lane * 4, sc_lds);
        if (wave == 0) lds_load<4>(down + 2 * (u64) ff + blockIdx.x * 256 + lane * 4, __builtin_amdgcn_readfirstlane(lds_offset(sv_out)));
        const u32* row0 = (const u32*) (down + 2 * (u64) ff + 2 * (u64) hidden + 4) + ((u64) kb * 8 * (hidden / 16) + blockIdx.x * 8) * EXL3_TILE_WORDS(K, false);
        const u64 pitch = (u64) (hidden / 16) * EXL3_TILE_WORDS(K, false);
        exl3_rows_issue<K, D>(row0, pitch, lane, wb_lds);
        wait_vm<R::loads>();
        const u16* sch = (const u16*) sc;
        const float s0 = f16_to_f32(sch[lane]), s1 = f16_to_f32(sch[lane + 64]);
        // a token's inverse scale and k_bias term wait in LDS for the lanes that hold the token's sums at the end
        float* ivs = (float*) (sc + 64);
#pragma unroll
        for (int r = 0; r < NMAX; r++) {
            if ((u32) r < n) {
                float a0 = (siluf_ref(gu[r][0]) * gu[r][2]) * s0, a1 = (siluf_ref(gu[r][1]) * gu[r][3]) * s1;
                const float c0 = (EXL3_KBIAS * 11.3137085f) * bits_f32(__builtin_amdgcn_readlane(f32_bits(a0), 0));
                wht128_wave(a0, a1, lane);
                const float i0 = exl3_put_a_rows<NMAX>(astrip, r, a0, a1, lane);
                if (lane == 0) {
                    ivs[r] = i0;
                    ivs[NMAX + r] = c0;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        exl3_wave_mma<K, LIN, NMAX>(row0, pitch, wring, wb_lds, astrip, n, lane, acc);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const u32 r = min(2 * (lane >> 4) + h, (u32) NMAX - 1);
            iv[h] = ivs[r];
            cr[h] = ivs[NMAX + r];
        }
    }
    __syncthreads();
    float* red = (float*) dyn;
    if (live) exl3_mma_to_red<LIN, NMAX>(red, wave, n, lane, acc, iv, cr);
    __syncthreads();
    const u32 nw = min(4u, kbs - blockIdx.z * 4);
    const u16* sv = (const u16*) sv_out;
    for (u32 r = wave; r < n; r += 4) {
        float a0 = 0.0f, a1 = 0.0f;
        for (u32 w = 0; w < nw; w++) {
            a0 += red[(w * NMAX + r) * 128 + lane];
            a1 += red[(w * NMAX + r) * 128 + lane + 64];
        }
        const u32 pair = (rec[4 + (r >> 1)] >> (16 * (r & 1))) & 0xffffu;
        if (gridDim.z == 1) {
            wht128_wave(a0, a1, lane);
            float* o = dn + (u64) pair * hidden + blockIdx.x * 128;
            __builtin_nontemporal_store(a0 * f16_to_f32(sv[lane]), &o[lane]);
            __builtin_nontemporal_store(a1 * f16_to_f32(sv[lane + 64]), &o[lane + 64]);
        } else {
            float* o = dn + ((u64) pair * gridDim.z + blockIdx.z) * hidden + blockIdx.x * 128;
            o[lane] = a0;
            o[lane + 64] = a1;
        }
    }
}

// Entry points: _mma_ the codebook's own f16 values, _lin_ the linearised form; the w variants take up to 8 tokens an item
// (batches of more than 4 rows), the others 4.  5 workgroups of 4 waves a CU: the register budget follows it.
#define EXL3_MMA_ENTRIES(K)                                                                                                            \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_gate_up_mma_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, \
                                                                                          u8* pbuf, u32 ioff, float* gup, u32 ne, u32 k, u32 m, u32 hidden, \
                                                                                          u32 ff) {                                      \
        verify_gate_up_mma_kernel<K, false, 4>(logits, ebase, estride, shbase, part, u, pbuf, ioff, gup, ne, k, m, hidden, ff);                     \
    }                                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_down_mma_exl3_##K(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf, \
                                                                                       u32 ioff, const float* gup, float* dn, u32 k, u32 m, u32 hidden, \
                                                                                       u32 ff, u32 zs) {                                 \
        verify_down_mma_kernel<K, false, 4>(ebase, estride, shbase, part, pbuf, ioff, gup, dn, k, m, hidden, ff, zs);                   \
    }
#define EXL3_MMAW_ENTRIES(K)                                                                                                            \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_gate_up_mmaw_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, \
                                                                                          u8* pbuf, u32 ioff, float* gup, u32 ne, u32 k, u32 m, u32 hidden, \
                                                                                          u32 ff) {                                      \
        verify_gate_up_mma_kernel<K, false, 8>(logits, ebase, estride, shbase, part, u, pbuf, ioff, gup, ne, k, m, hidden, ff);                     \
    }                                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_down_mmaw_exl3_##K(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf, \
                                                                                       u32 ioff, const float* gup, float* dn, u32 k, u32 m, u32 hidden, \
                                                                                       u32 ff, u32 zs) {                                 \
        verify_down_mma_kernel<K, false, 8>(ebase, estride, shbase, part, pbuf, ioff, gup, dn, k, m, hidden, ff, zs);                   \
    }
#define EXL3_LIN_ENTRIES(K)                                                                                                            \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_gate_up_lin_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, \
                                                                                          u8* pbuf, u32 ioff, float* gup, u32 ne, u32 k, u32 m, u32 hidden, \
                                                                                          u32 ff) {                                      \
        verify_gate_up_mma_kernel<K, true, 4>(logits, ebase, estride, shbase, part, u, pbuf, ioff, gup, ne, k, m, hidden, ff);                     \
    }                                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_down_lin_exl3_##K(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf, \
                                                                                       u32 ioff, const float* gup, float* dn, u32 k, u32 m, u32 hidden, \
                                                                                       u32 ff, u32 zs) {                                 \
        verify_down_mma_kernel<K, true, 4>(ebase, estride, shbase, part, pbuf, ioff, gup, dn, k, m, hidden, ff, zs);                   \
    }
#define EXL3_LINW_ENTRIES(K)                                                                                                            \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_gate_up_linw_exl3_##K(const float* logits, u64 ebase, u64 estride, u64 shbase, u32 part, const float* u, \
                                                                                          u8* pbuf, u32 ioff, float* gup, u32 ne, u32 k, u32 m, u32 hidden, \
                                                                                          u32 ff) {                                      \
        verify_gate_up_mma_kernel<K, true, 8>(logits, ebase, estride, shbase, part, u, pbuf, ioff, gup, ne, k, m, hidden, ff);                     \
    }                                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256, 5) verify_down_linw_exl3_##K(u64 ebase, u64 estride, u64 shbase, u32 part, const u8* pbuf, \
                                                                                       u32 ioff, const float* gup, float* dn, u32 k, u32 m, u32 hidden, \
                                                                                       u32 ff, u32 zs) {                                 \
        verify_down_mma_kernel<K, true, 8>(ebase, estride, shbase, part, pbuf, ioff, gup, dn, k, m, hidden, ff, zs);                   \
    }
EXL3_MMA_ENTRIES(1)
EXL3_MMA_ENTRIES(2)
EXL3_MMA_ENTRIES(3)
EXL3_MMA_ENTRIES(4)
EXL3_MMA_ENTRIES(5)
EXL3_MMA_ENTRIES(6)
EXL3_MMA_ENTRIES(7)
EXL3_MMA_ENTRIES(8)
EXL3_MMAW_ENTRIES(1)
EXL3_MMAW_ENTRIES(2)
EXL3_MMAW_ENTRIES(3)
EXL3_MMAW_ENTRIES(4)
EXL3_MMAW_ENTRIES(5)
EXL3_MMAW_ENTRIES(6)
EXL3_MMAW_ENTRIES(7)
EXL3_MMAW_ENTRIES(8)
EXL3_LIN_ENTRIES(1)
EXL3_LIN_ENTRIES(2)
EXL3_LIN_ENTRIES(3)
EXL3_LIN_ENTRIES(4)
EXL3_LIN_ENTRIES(5)
EXL3_LIN_ENTRIES(6)
EXL3_LIN_ENTRIES(7)
EXL3_LIN_ENTRIES(8)
EXL3_LINW_ENTRIES(1)
EXL3_LINW_ENTRIES(2)
EXL3_LINW_ENTRIES(3)
EXL3_LINW_ENTRIES(4)
EXL3_LINW_ENTRIES(5)
EXL3_LINW_ENTRIES(6)
EXL3_LINW_ENTRIES(7)
EXL3_LINW_ENTRIES(8)

// ------------------------------------------------------------------------ the prefill chunk of an EXL3 layer (matrix cores)
// A chunk's tokens grouped by expert (prefill_group in kernels/prefill.hip: runs of up to XPF_TOK(K) (token, rank) pairs of
// one expert are a work item) through gate/up, the activation and down with the item's tokens on the columns of the matrix
// instruction: an expert's weights are decoded once for all tokens of an item (the reference's mma_grouped_exl3_pre_K,
// kernels/exl3.cu:684,704,724, with groups of 64, session.rs:5159-5189).  The rotations of the format run on the matrix
// cores too: H (x * suh) is a product with the 128 x 128 matrix of signs, whose 16 x 16 x 16 operands a lane makes from
// its own lane number (H[i][j] = (-1)^popcount(i & j): a tile of it is a per-lane pattern times the parity of the two
// tile numbers).  Every product here has the tokens on the columns (operand B, lane 16 a + n: token n, inputs 4 a .. 4 a
// + 3) and its result on the same lanes as (token n, outputs 4 a .. 4 a + 3): a result is the next product's operand as
// it lies, nothing is transposed.  Inputs of a rotation ride as an f16 high and an f16 low part, scaled by a power of two
// per token; the rotated values as single f16 values (the reference converts to f16 unscaled); weights are the
// codebook's own f16 values; sums are f32.  Against the exact arithmetic the f16 roundings of the activations cost about
// 4e-4 relative L2 of a layer's output (bound of the path: 1e-3).
//
// Three launches a layer.  1: (item, gate | up, share z of the inputs): the x rotation and the products, raw partial sums
// to memory.  2: (item, tile of 16 tokens): the partial sums added up, the output-side transforms and scales of gate and
// up, act = silu(gate) * up, its rotation into the down projection's basis, left as the f16 operand rows of launch 3.
// 3: (item, four 128-column blocks of hidden): the products, the output side, the pairs' rows of the layer's result.

// Tokens of a work item: as many tiles of 16 as leave room for two workgroups' LDS on a compute unit (the operand rows of four
// 128-blocks, 1 KiB a token, and the four waves' rings of trellis rows).
#define XPF_NT(K) ((K) <= 7 ? 3 : 2)
// Rows of a wave's ring: what is left of half a compute unit's LDS (rows of 256, 512, 1024 (K = 3, 4) or 256 K bytes)
#define XPF_D(K) ((K) <= 2 ? 8 : (K) <= 5 ? 6 : 4)
#define XPF_TOK(K) (16 * XPF_NT(K))

// The lane's share of a sign tile of H: element q of the pair is H[16 i + n][16 j + 4 a + q] (= H[16 j + 4 a + q][16 i + n])
// for tile numbers of even popcount(i & j) (a = lane / 16, n = lane % 16); the other tiles are the negative.
__device__ __forceinline__ void xpf_sign_tile(u32 lane, u32 (&hop)[2]) {
    const u32 n = lane & 15, a = lane >> 4;
    u32 h[4];
#pragma unroll
    for (u32 q = 0; q < 4; q++) h[q] = (__builtin_popcount((4 * a + q) & n) & 1) ? 0xbc00u : 0x3c00u;   // -1.0 : +1.0
    hop[0] = h[0] | (h[1] << 16);
    hop[1] = h[2] | (h[3] << 16);
}

// rot[ct][q] = sum over the 128 inputs i of H[16 ct + 4 a + q][i] v[i] for the lane's token (n = lane % 16 of the tile): v
// comes as load4(ks) = the token's inputs 16 ks + 4 a .. + 3 (already times the input scales and the token's power of two).
// An input goes in as an f16 high and an f16 low part (22 bits of it; the signs are exact, the sums f32): the rotation
// itself adds no rounding that matters.
template <class F>
__device__ __forceinline__ void xpf_rotate_tile(F&& load4, const u32 (&hop)[2], f32x4 (&rot)[8]) {
#pragma unroll
    for (int ct = 0; ct < 8; ct++) rot[ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // the high and the low parts share one 32-deep matrix instruction: its operands are the sign tile twice and the two parts
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    typedef u32 u32x4v __attribute__((ext_vector_type(4)));
    typedef u32 u32x2 __attribute__((ext_vector_type(2)));
    const f16x8 hp = __builtin_bit_cast(f16x8, u32x4v{hop[0], hop[1], hop[0], hop[1]});
    const f16x8 hn = __builtin_bit_cast(f16x8, u32x4v{hop[0] ^ 0x80008000u, hop[1] ^ 0x80008000u, hop[0] ^ 0x80008000u, hop[1] ^ 0x80008000u});
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        const f32x4 v = load4(ks);
        const f16x4 av = {(_Float16) v[0], (_Float16) v[1], (_Float16) v[2], (_Float16) v[3]};
        const f16x4 al = {(_Float16) (v[0] - (float) av[0]), (_Float16) (v[1] - (float) av[1]), (_Float16) (v[2] - (float) av[2]), (_Float16) (v[3] - (float) av[3])};
        const u32x2 ab = __builtin_bit_cast(u32x2, av), lb = __builtin_bit_cast(u32x2, al);
        const f16x8 parts = __builtin_bit_cast(f16x8, u32x4v{ab[0], ab[1], lb[0], lb[1]});
#pragma unroll
        for (int ct = 0; ct < 8; ct++) {
            const bool neg = __builtin_popcount(ks & ct) & 1;
            rot[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(neg ? hn : hp, parts, rot[ct], 0, 0, 0);
        }
    }
}

// The largest magnitude of the lane's token's 128 values: the lane's 32 of them, then the lanes + 16, + 32, + 48.
__device__ __forceinline__ float xpf_token_max(const f32x4 (&v)[8], u32 lane) {
    float m = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 8; ks++)
#pragma unroll
        for (int q = 0; q < 4; q++) m = fmaxf(m, __builtin_fabsf(v[ks][q]));
    m = fmaxf(m, lane_xor<16>(m, lane));
    return fmaxf(m, lane_xor<32>(m, lane));
}

// A 128-block of the lane's token through H, its values brought into f16's range for the product by the token's own power
// of two and back afterwards (exact both ways): rot = H v.
__device__ __forceinline__ void xpf_rotate_scaled(const f32x4 (&v)[8], const u32 (&hop)[2], f32x4 (&rot)[8], u32 lane) {
    float scale, inv;
    pow2_scale_of(f32_bits(xpf_token_max(v, lane)), scale, inv);
    xpf_rotate_tile([&](int ks) { return v[ks] * scale; }, hop, rot);
#pragma unroll
    for (int ct = 0; ct < 8; ct++) rot[ct] *= inv;
}

// The operand rows of the products.  A token tile's rows: [tile row i of the item's up to 32 (block * 8 + ct)][token n][16
// values in the order the decode lanes take them], 512 bytes a tile row; the tiles of an item follow each other.  The lane
// holds the values 4 a + q of tile row ct of its token: slots 8 (a & 1) + 2 (a >> 1) + {0, 1} and + 4 of that (exl3_aslot).
// rot must be bounded by 2^22 (inputs scaled to below 2^15, 128 terms): the stored value is f16(rot / 128).
#define XPF_TILE_U16 (32 * 256)      // u16 of a token tile's operand rows (four 128-blocks)
__device__ __forceinline__ void xpf_put_rows(u16* tile, u32 block, const f32x4 (&rot)[8], u32 lane) {
    const u32 n = lane & 15, a = lane >> 4;
    u32* at = (u32*) (tile + (block * 8) * 256 + n * 16 + 8 * (a & 1) + 2 * (a >> 1));
#pragma unroll
    for (int ct = 0; ct < 8; ct++) {
        const f16x2 lo = {(_Float16) (rot[ct][0] * 0.0078125f), (_Float16) (rot[ct][1] * 0.0078125f)};
        const f16x2 hi = {(_Float16) (rot[ct][2] * 0.0078125f), (_Float16) (rot[ct][3] * 0.0078125f)};
        at[ct * 128] = __builtin_bit_cast(u32, lo);
        at[ct * 128 + 2] = __builtin_bit_cast(u32, hi);
    }
}
// what undoes the 1 / 128 of the stored values and applies the transform's 1 / sqrt(128)
#define XPF_UNSCALE 11.3137085f

// The products of one wave: `nrows` tile rows of its 128-column block (the stream starts at row0, its first rows already
// requested) against the operand rows of NT token tiles at xa; acc[T][c][q] = output 16 c + 4 a + q of token 16 T + n.
template <int K, int NT>
__device__ __forceinline__ void xpf_wave_products_of(const u32* __restrict__ row0, u64 pitch, u32 nrows, const u32* wb, u32 lds, const u16* xa, u32 lane,
                                                     f32x4 (&acc)[XPF_NT(K)][8]) {
    constexpr int D = XPF_D(K);
    typedef Exl3Rows<K, D> R;
    constexpr int stride = R::stride, ur = R::unit_rows;
    constexpr bool one_shift = 16 + 3 * K <= 32;
    const u32 n16 = lane & 15, a = lane >> 4;
    const u32 t0 = 32 * (n16 & 7) + 8 * a + 4 * (n16 >> 3);
    auto window = [&](u32 e, u32& om, u32& op, u32& sh) {
        const u32 jp = (e - 1) >> 5, jm = (jp + 8 * K - 1) % (8 * K);
        sh = 31 - ((e - 1) & 31);
        om = (jm / K) * stride + jm % K;
        op = (jp / K) * stride + jp % K;
    };
    u32 om1, op1, sh1, om0 = 0, op0 = 0, sh0 = 0;
    window((t0 + 4) * K, om1, op1, sh1);
    if constexpr (!one_shift) window((t0 + 2) * K, om0, op0, sh0);
#pragma unroll
    for (int T = 0; T < NT; T++)
#pragma unroll
        for (int c = 0; c < 8; c++) acc[T][c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const u16* xa0 = xa + n16 * 16 + 4 * a;
    typedef u32 u32x2 __attribute__((ext_vector_type(2)));
    if constexpr (one_shift && ur == 1) {
        // Two tile rows a step: a lane's 4 + 4 weights of the rows' tiles are one operand of the 32-deep matrix instruction
        // (the contraction runs over both rows' 16 inputs; which of them a lane holds does not matter as long as the token
        // operand is put together the same way), which halves the matrix instructions and their issue slots.
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
        typedef u32 u32x4v __attribute__((ext_vector_type(4)));
#pragma unroll 1
        for (u32 i = 0; i < nrows; i += 2) {   // a stream is a whole number of 8-row blocks
            u32 w1[2][8][2];
            u32x2 xv[2][NT];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const u32 r = i + h;
                exl3_rows_wait<K, D>(r + D > nrows ? r + D - nrows : 0);
                const u32* row = wb + (r % D) * R::row_words;
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    w1[h][c][0] = row[c * 8 * stride + om1];
                    w1[h][c][1] = row[c * 8 * stride + op1];
                }
#pragma unroll
                for (int T = 0; T < NT; T++) xv[h][T] = *(const u32x2*) (xa0 + T * XPF_TILE_U16 + r * 256);
                if (r + D < nrows) {
                    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the row's words are in registers, its slot can take the row D further on
                    exl3_unit_issue<K, D>(row0, pitch, r + D, lane, lds);
                }
            }
#pragma unroll
            for (int c = 0; c < 8; c++) {
                u32 b[2][2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const u32 hi = __builtin_amdgcn_alignbit(w1[h][c][0], w1[h][c][1], sh1);
                    const u32 s0 = __builtin_amdgcn_ubfe(hi, 3 * K, 16), s1 = __builtin_amdgcn_ubfe(hi, 2 * K, 16);
                    const u32 s2 = __builtin_amdgcn_ubfe(hi, K, 16), s3 = hi & 0xffffu;
                    b[h][0] = __builtin_bit_cast(u32, exl3_cb2_pair(s0, s1));
                    b[h][1] = __builtin_bit_cast(u32, exl3_cb2_pair(s2, s3));
                }
                const f16x8 bv = __builtin_bit_cast(f16x8, u32x4v{b[0][0], b[0][1], b[1][0], b[1][1]});
#pragma unroll
                for (int T = 0; T < NT; T++) {
                    const f16x8 tv = __builtin_bit_cast(f16x8, u32x4v{xv[0][T][0], xv[0][T][1], xv[1][T][0], xv[1][T][1]});
                    acc[T][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bv, tv, acc[T][c], 0, 0, 0);
                }
            }
        }
        return;
    }
#pragma unroll 1
    for (u32 i = 0; i < nrows; i++) {
        exl3_rows_wait<K, D>(i + D > nrows ? i + D - nrows : 0);
        const u32* row = wb + (i % D) * R::row_words;
        u32 w1[8][2], w0[8][2];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            w1[c][0] = row[c * 8 * stride + om1];
            w1[c][1] = row[c * 8 * stride + op1];
            if constexpr (!one_shift) {
                w0[c][0] = row[c * 8 * stride + om0];
                w0[c][1] = row[c * 8 * stride + op0];
            }
        }
        f16x4 xv[NT];
#pragma unroll
        for (int T = 0; T < NT; T++) xv[T] = __builtin_bit_cast(f16x4, *(const u32x2*) (xa0 + T * XPF_TILE_U16 + i * 256));
        if ((i + 1) % ur == 0 && i + D + 1 - ur < nrows) {
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the row's words are in registers, its slot can take the row D further on
            exl3_unit_issue<K, D>(row0, pitch, i + D + 1 - ur, lane, lds);
        }
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const u32 hi = __builtin_amdgcn_alignbit(w1[c][0], w1[c][1], sh1);
            u32 s0, s1;
            if constexpr (one_shift) {
                s0 = __builtin_amdgcn_ubfe(hi, 3 * K, 16);
                s1 = __builtin_amdgcn_ubfe(hi, 2 * K, 16);
            } else {
                const u32 lo = __builtin_amdgcn_alignbit(w0[c][0], w0[c][1], sh0);
                s0 = __builtin_amdgcn_ubfe(lo, K, 16);
                s1 = lo & 0xffffu;
            }
            const u32 s2 = __builtin_amdgcn_ubfe(hi, K, 16), s3 = hi & 0xffffu;
            const f16x2 b01 = exl3_cb2_pair(s0, s1), b23 = exl3_cb2_pair(s2, s3);
            const f16x4 bv = {b01[0], b01[1], b23[0], b23[1]};
#pragma unroll
            for (int T = 0; T < NT; T++) acc[T][c] = __builtin_amdgcn_mfma_f32_16x16x16f16(bv, xv[T], acc[T][c], 0, 0, 0);
        }
    }
}

// One loop for every number of token tiles: the choice is made once, outside the loop.
template <int K>
__device__ __forceinline__ void xpf_wave_products(const u32* __restrict__ row0, u64 pitch, u32 nrows, const u32* wb, u32 lds, const u16* xa, u32 ntiles,
                                                  u32 lane, f32x4 (&acc)[XPF_NT(K)][8]) {
    if (ntiles == 1) xpf_wave_products_of<K, 1>(row0, pitch, nrows, wb, lds, xa, lane, acc);
    else if (ntiles == 2) xpf_wave_products_of<K, 2>(row0, pitch, nrows, wb, lds, xa, lane, acc);
    else if constexpr (XPF_NT(K) >= 3) xpf_wave_products_of<K, 3>(row0, pitch, nrows, wb, lds, xa, lane, acc);
}

// The output side of a wave's block for the lane's token: v[c][q] = output 16 c + 4 a + q goes through the 128-point
// transform.  Five of its seven stages are between the lane's own registers; the two over the lane number's bits 4 and 5 are
// swaps of register halves between the lanes (one swap serves two registers), after which the lane holds OTHER outputs of
// its token: register c, element q is output xpf_out_col(c, lane) + q.
__device__ __forceinline__ u32 xpf_out_col(u32 c, u32 lane) { return 64 * (c >> 2) + 32 * ((lane >> 4) & 1) + 16 * (lane >> 5) + 8 * (c & 1) + 4 * ((c >> 1) & 1); }
__device__ __forceinline__ void xpf_output_side(f32x4 (&v)[8]) {
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const float t0 = v[c][0] + v[c][1], t1 = v[c][0] - v[c][1], t2 = v[c][2] + v[c][3], t3 = v[c][2] - v[c][3];
        v[c] = f32x4{t0 + t2, t1 + t3, t0 - t2, t1 - t3};
    }
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
        for (int c = 0; c < 8; c++)
            if (!(c & h)) {
                const f32x4 s = v[c] + v[c + h], d = v[c] - v[c + h];
                v[c] = s;
                v[c + h] = d;
            }
    // lane bit 5 (output bit 3): the upper half of register c and the lower half of register c + 1 change places; then both lanes
    // of a pair hold the two ends of one butterfly.  Register c keeps the sum (bit 3 clear), c + 1 the difference; the lane's
    // bit 5 now says which of the two registers' outputs (output bit 4) it holds.
#pragma unroll
    for (int c = 0; c < 8; c += 2)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const auto r = __builtin_amdgcn_permlane32_swap(f32_bits(v[c][q]), f32_bits(v[c + 1][q]), false, false);
            v[c][q] = bits_f32(r[0]) + bits_f32(r[1]);
            v[c + 1][q] = bits_f32(r[0]) - bits_f32(r[1]);
        }
    // lane bit 4 (output bit 2) with the registers c and c + 2 (output bit 5) likewise
#pragma unroll
    for (int c = 0; c < 8; c++)
        if (!(c & 2)) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const auto r = __builtin_amdgcn_permlane16_swap(f32_bits(v[c][q]), f32_bits(v[c + 2][q]), false, false);
                v[c][q] = bits_f32(r[0]) + bits_f32(r[1]);
                v[c + 2][q] = bits_f32(r[0]) - bits_f32(r[1]);
            }
        }
}

// Shared set-up of the launches: the item, its pairs and rows (tok = the most pairs of an item).  Returns the number of the
// item's pairs (0: no such item).
__device__ __forceinline__ u32 xpf_item(const u32* __restrict__ offs, const u32* __restrict__ list, const u32* __restrict__ items, u32 item, u32 ne, bool has_shared,
                                        u32 k, u32 npairs, u32 tok, u32* s_pairs, u32* s_rows, u32& e) {
    if (item >= items[0]) return 0;
    e = items[1 + 2 * item];
    const u32 t0 = items[2 + 2 * item];
    if (e == ne && !has_shared) return 0;
    const u32 first = offs[e], nt = min(tok, offs[e + 1] - first - t0);
    if (threadIdx.x < tok) {
        const u32 p = list[first + t0 + min(threadIdx.x, nt - 1)];   // a place past the item's end repeats its last pair: loads stay in bounds, results are dropped
        s_pairs[threadIdx.x] = p;
        s_rows[threadIdx.x] = p < npairs ? p / k : p - npairs;
    }
    return nt;
}

// LDS of a workgroup of launches 1 and 3, in words: the operand rows of the item's token tiles, the four waves' rings, the
// item's pairs and rows, the waves' token maxima, the tokens' factors.
#define XPF_LDS_WORDS(ring, tok) ((tok) / 16 * (XPF_TILE_U16 / 2) + 4 * (ring) + 2 * (tok) + 4 * (tok) + (tok))

// Launch 1: item blockIdx.x, sel = blockIdx.y / zs (gate, up), z = blockIdx.y % zs: the inputs' 128-blocks 4 z .. 4 z + 3.
// Wave w rotates block 4 z + w of the item's tokens, then takes the 128-column blocks w, w + 4, .. of ff over the four input
// blocks; raw partial sums gup[((sel * NP + pair) * zs + z)][ff] (NP = npairs + the shared expert's rows): the output side
// is launch 2's.  grid = (bound on the items, 2 zs), block 256, dynamic LDS 4 XPF_LDS_WORDS.
template <int K>
__device__ __forceinline__ void prefill_gate_up_exl3_kernel(const u64* __restrict__ eaddr, const u64* __restrict__ sh_addr, const u32* __restrict__ offs,
                                                            const u32* __restrict__ list, const u32* __restrict__ items, const float* __restrict__ x,
                                                            float* __restrict__ gup, u32 ne, u32 k, u32 npairs, u32 NP, u32 hidden, u32 ff) {
    typedef Exl3Rows<K, XPF_D(K)> R;
    constexpr u32 TOK = XPF_TOK(K);
    extern __shared__ __attribute__((aligned(16))) u32 dyn[];
    u16* arows = (u16*) dyn;                                  // [token tile][block of the four][tile row][token][16]
    u32* rings = dyn + XPF_NT(K) * (XPF_TILE_U16 / 2);
    u32* s_pairs = rings + 4 * R::words;
    u32* s_rows = s_pairs + TOK;
    float* s_max = (float*) (s_rows + TOK);                   // [wave][token]
    float* s_inv = s_max + 4 * TOK;                           // [token]
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32 kbs = hidden / 128, zs = (kbs + 3) / 4, sel = blockIdx.y / zs, z = blockIdx.y - sel * zs;
    u32 e;
    const u32 nt = xpf_item(offs, list, items, blockIdx.x, ne, sh_addr != nullptr, k, npairs, TOK, s_pairs, s_rows, e);
    if (nt == 0) return;
    const u32 ntiles = (nt + 15) / 16;
    const u8* bp = (const u8*) (e < ne ? eaddr[(u64) sel * ne + e] : sh_addr[sel]);
    const u32 kb = 4 * z + wave, nkb = min(4u, kbs - 4 * z);
    __syncthreads();                                          // the item's pairs and rows are written
    typedef u16 u16x4 __attribute__((ext_vector_type(4)));
    float sc[8][4];
    if (wave < nkb) {
        // the largest input of every token over the block: the token's power of two must be one for the workgroup's four blocks
        const u16* suh = (const u16*) bp + kb * 128 + 4 * (lane >> 4);
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            const u16x4 s4 = *(const u16x4*) (suh + 16 * ks);
#pragma unroll
            for (int q = 0; q < 4; q++) sc[ks][q] = f16_to_f32(s4[q]);
        }
        for (u32 T = 0; T < ntiles; T++) {
            const float* xr = x + (u64) s_rows[16 * T + (lane & 15)] * hidden + kb * 128 + 4 * (lane >> 4);
            f32x4 xv[8];
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                xv[ks] = *(const f32x4*) (xr + 16 * ks);
#pragma unroll
                for (int q = 0; q < 4; q++) xv[ks][q] *= sc[ks][q];
            }
            const float m = xpf_token_max(xv, lane);
            if (lane < 16) s_max[wave * TOK + 16 * T + lane] = m;
        }
    }
    __syncthreads();
    if (wave < nkb) {
        u32 hop[2];
        xpf_sign_tile(lane, hop);
        for (u32 T = 0; T < ntiles; T++) {
            const u32 t = 16 * T + (lane & 15);
            float m = 0.0f;
            for (u32 w = 0; w < nkb; w++) m = fmaxf(m, s_max[w * TOK + t]);
            float scale, iv;
            pow2_scale_of(f32_bits(m), scale, iv);
            if (wave == 0 && lane < 16) s_inv[t] = iv * XPF_UNSCALE;
            const float* xr = x + (u64) s_rows[t] * hidden + kb * 128 + 4 * (lane >> 4);   // the second read comes from the caches
            f32x4 rot[8];
            xpf_rotate_tile(
                [&](int ks) {
                    f32x4 v = *(const f32x4*) (xr + 16 * ks);
#pragma unroll
                    for (int q = 0; q < 4; q++) v[q] = (v[q] * sc[ks][q]) * scale;
                    return v;
                },
                hop, rot);
            xpf_put_rows(arows + T * XPF_TILE_U16, wave, rot, lane);
        }
    }
    __syncthreads();
    const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(rings + wave * R::words));
    const u64 pitch = (u64) (ff / 16) * EXL3_TILE_WORDS(K, false);
    for (u32 cb = wave; cb < ff / 128; cb += 4) {
        const u32* row0 = (const u32*) (bp + 2 * (u64) hidden + 2 * (u64) ff + 4) + ((u64) (4 * z) * 8 * (ff / 16) + cb * 8) * EXL3_TILE_WORDS(K, false);
        exl3_rows_issue<K, XPF_D(K)>(row0, pitch, lane, wb_lds);     // a stream has at least 8 rows
        f32x4 acc[XPF_NT(K)][8];
        xpf_wave_products<K>(row0, pitch, 8 * nkb, rings + wave * R::words, wb_lds, arows, ntiles, lane, acc);
#pragma unroll
        for (int T = 0; T < XPF_NT(K); T++) {
            if ((u32) T >= ntiles) break;
            const u32 t = 16 * T + (lane & 15);
            const float iv = s_inv[t];
            if (t < nt) {
                float* o = gup + (((u64) sel * NP + s_pairs[t]) * zs + z) * ff + cb * 128 + 4 * (lane >> 4);
#pragma unroll
                for (int c = 0; c < 8; c++) *(f32x4*) (o + 16 * c) = acc[T][c] * iv;
            }
        }
    }
}

// Launch 2 (one kernel for every rate): tile blockIdx.y (16 tokens) of item blockIdx.x.  Wave w takes block w of ff (ff <=
// 512: four blocks): adds up launch 1's partial sums of gate and up, puts both through their output sides (transform, output
// scales), act = silu(gate) * up times the down projection's input scales, rotated, and leaves it as operand rows for
// launch 3: arows[item * tok / 16 + tile] = a token tile's rows (XPF_TILE_U16), ainv[item * tok + token] = what undoes the
// token's power of two.  grid = (bound on the items, tok / 16), block 256.
extern "C" __global__ void __launch_bounds__(256, 2) prefill_act_exl3(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list, const u32* items,
                                                                      const float* gup, u16* arows, float* ainv, u32 ne, u32 k, u32 npairs, u32 NP,
                                                                      u32 hidden, u32 ff, u32 zs, u32 tok) {
    __shared__ u32 s_pairs[64], s_rows[64];
    __shared__ float s_max[4 * 16];
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32 kbs = ff / 128, T = blockIdx.y;                  // kbs: at most 4
    u32 e;
    const u32 nt = xpf_item(offs, list, items, blockIdx.x, ne, sh_addr != nullptr, k, npairs, tok, s_pairs, s_rows, e);
    if (16 * T >= nt) return;
    __syncthreads();
    const u8* bg = (const u8*) (e < ne ? eaddr[e] : sh_addr[0]);
    const u8* bu = (const u8*) (e < ne ? eaddr[(u64) ne + e] : sh_addr[1]);
    const u8* bd = (const u8*) (e < ne ? eaddr[2ull * ne + e] : sh_addr[2]);
    typedef u16 u16x4 __attribute__((ext_vector_type(4)));
    u32 hop[2];
    xpf_sign_tile(lane, hop);
    f32x4 act[8];
    float m = 0.0f;
    if (wave < kbs) {
        const u32 pair = s_pairs[16 * T + (lane & 15)], at = wave * 128 + 4 * (lane >> 4);
        const float* pg = gup + ((u64) pair * zs) * ff + at;
        const float* pu = gup + (((u64) NP + pair) * zs) * ff + at;
        f32x4 g[8], u[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            g[ks] = *(const f32x4*) (pg + 16 * ks);
            u[ks] = *(const f32x4*) (pu + 16 * ks);
        }
        for (u32 zz = 1; zz < zs; zz++)
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                g[ks] += *(const f32x4*) (pg + (u64) zz * ff + 16 * ks);
                u[ks] += *(const f32x4*) (pu + (u64) zz * ff + 16 * ks);
            }
        f32x4 gr[8];
        xpf_rotate_scaled(g, hop, gr, lane);
        xpf_rotate_scaled(u, hop, g, lane);                    // g: the rotated up from here on
        const u16* svg = (const u16*) (bg + 2 * (u64) hidden) + at;
        const u16* svu = (const u16*) (bu + 2 * (u64) hidden) + at;
        const u16* suh = (const u16*) bd + at;
#pragma unroll
        for (int ct = 0; ct < 8; ct++) {
            const u16x4 a4 = *(const u16x4*) (svg + 16 * ct), b4 = *(const u16x4*) (svu + 16 * ct), c4 = *(const u16x4*) (suh + 16 * ct);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float gate = gr[ct][q] * (f16_to_f32(a4[q]) * 0.08838835f), up = g[ct][q] * (f16_to_f32(b4[q]) * 0.08838835f);
                act[ct][q] = (siluf_ref(gate) * up) * f16_to_f32(c4[q]);
            }
        }
        m = xpf_token_max(act, lane);
        if (lane < 16) s_max[wave * 16 + lane] = m;
    }
    __syncthreads();
    if (wave >= kbs) return;
    m = 0.0f;
    for (u32 w = 0; w < kbs; w++) m = fmaxf(m, s_max[w * 16 + (lane & 15)]);
    float scale, iv;
    pow2_scale_of(f32_bits(m), scale, iv);
    if (wave == 0 && lane < 16) ainv[(u64) blockIdx.x * tok + 16 * T + lane] = iv * XPF_UNSCALE;
    f32x4 rot[8];
    xpf_rotate_tile([&](int ks) { return act[ks] * scale; }, hop, rot);
    xpf_put_rows(arows + ((u64) blockIdx.x * (tok / 16) + T) * XPF_TILE_U16, wave, rot, lane);
}

// Launch 3: item blockIdx.x, 128-column blocks 4 blockIdx.y + w of hidden for wave w: the products of the item's operand rows
// (copied from launch 2's into LDS, wave w its block w of every tile) over the ff / 128 input blocks and the output side:
// eo[pair][hidden].  grid = (bound on the items, ceil(hidden / 512)), block 256, dynamic LDS 4 XPF_LDS_WORDS.
template <int K>
__device__ __forceinline__ void prefill_down_exl3_kernel(const u64* __restrict__ eaddr, const u64* __restrict__ sh_addr, const u32* __restrict__ offs,
                                                         const u32* __restrict__ list, const u32* __restrict__ items, const u16* __restrict__ arows_g,
                                                         const float* __restrict__ ainv, float* __restrict__ eo, u32 ne, u32 k, u32 npairs, u32 hidden, u32 ff) {
    typedef Exl3Rows<K, XPF_D(K)> R;
    constexpr u32 TOK = XPF_TOK(K);
    extern __shared__ __attribute__((aligned(16))) u32 dyn[];
    u16* arows = (u16*) dyn;
    u32* rings = dyn + XPF_NT(K) * (XPF_TILE_U16 / 2);
    u32* s_pairs = rings + 4 * R::words;
    u32* s_rows = s_pairs + TOK;
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const u32 kbs = ff / 128;                                  // at most 4
    u32 e;
    const u32 nt = xpf_item(offs, list, items, blockIdx.x, ne, sh_addr != nullptr, k, npairs, TOK, s_pairs, s_rows, e);
    if (nt == 0) return;
    const u32 ntiles = (nt + 15) / 16;
    const u8* down = (const u8*) (e < ne ? eaddr[2ull * ne + e] : sh_addr[2]);
    const u32 cb = 4 * blockIdx.y + wave;
    const bool live = cb < hidden / 128;
    // what undoes the powers of two of the lane's tokens (the only ordinary loads: consumed before the burst)
    float iv[XPF_NT(K)];
#pragma unroll
    for (int T = 0; T < XPF_NT(K); T++) iv[T] = (u32) T < ntiles ? ainv[(u64) blockIdx.x * TOK + 16 * T + (lane & 15)] : 0.0f;
#pragma unroll
    for (int T = 0; T < XPF_NT(K); T++) asm volatile("" : "+v"(iv[T]));
    const u32 wb_lds = __builtin_amdgcn_readfirstlane(lds_offset(rings + wave * R::words));
    if (wave < kbs) {
        // block `wave` of every live tile: 8 tile rows of 512 bytes, 1 KiB a load
        for (u32 T = 0; T < ntiles; T++) {
            const u8* src = (const u8*) (arows_g + ((u64) blockIdx.x * XPF_NT(K) + T) * XPF_TILE_U16 + wave * 8 * 256);
            const u32 dst = __builtin_amdgcn_readfirstlane(lds_offset(arows + T * XPF_TILE_U16 + wave * 8 * 256));
#pragma unroll
            for (int i = 0; i < 4; i++) lds_load<16>(src + i * 1024 + lane * 16, dst + i * 1024);
        }
    }
    const u64 pitch = (u64) (hidden / 16) * EXL3_TILE_WORDS(K, false);
    const u32* row0 = (const u32*) (down + 2 * (u64) ff + 2 * (u64) hidden + 4) + (u64) (live ? cb : 0) * 8 * EXL3_TILE_WORDS(K, false);
    if (live) {
        exl3_rows_issue<K, XPF_D(K)>(row0, pitch, lane, wb_lds);
        wait_vm<R::loads>();                                  // this wave's operand rows have landed (its ring may still be on its way)
    } else wait_vm<0>();
    __syncthreads();                                          // every wave's operand rows, and the item's pairs
    if (!live) return;
    f32x4 acc[XPF_NT(K)][8];
    xpf_wave_products<K>(row0, pitch, 8 * kbs, rings + wave * R::words, wb_lds, arows, ntiles, lane, acc);
    typedef u16 u16x4 __attribute__((ext_vector_type(4)));
    const u16* svh = (const u16*) (down + 2 * (u64) ff) + cb * 128;
    f32x4 sv[8];
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const u16x4 s4 = *(const u16x4*) (svh + xpf_out_col(c, lane));
#pragma unroll
        for (int q = 0; q < 4; q++) sv[c][q] = f16_to_f32(s4[q]) * 0.08838835f;
    }
#pragma unroll
    for (int T = 0; T < XPF_NT(K); T++) {
        if ((u32) T >= ntiles) break;
#pragma unroll
        for (int c = 0; c < 8; c++) acc[T][c] *= iv[T];
        xpf_output_side(acc[T]);
        const u32 t = 16 * T + (lane & 15);
        if (t < nt) {
            float* o = eo + (u64) s_pairs[t] * hidden + cb * 128;
#pragma unroll
            for (int c = 0; c < 8; c++) *(f32x4*) (o + xpf_out_col(c, lane)) = acc[T][c] * sv[c];
        }
    }
}

#define EXL3_PREFILL_ENTRIES(K)                                                                                                          \
    extern "C" __global__ void __launch_bounds__(256, 2) prefill_gate_up_exl3_##K(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list, \
                                                                                   const u32* items, const float* x, float* gup, u32 ne, u32 k, u32 npairs, \
                                                                                   u32 NP, u32 hidden, u32 ff) {                         \
        prefill_gate_up_exl3_kernel<K>(eaddr, sh_addr, offs, list, items, x, gup, ne, k, npairs, NP, hidden, ff);                        \
    }                                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256, 2) prefill_down_exl3_##K(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list, \
                                                                                const u32* items, const u16* arows, const float* ainv, float* eo, u32 ne, \
                                                                                u32 k, u32 npairs, u32 hidden, u32 ff) {                 \
        prefill_down_exl3_kernel<K>(eaddr, sh_addr, offs, list, items, arows, ainv, eo, ne, k, npairs, hidden, ff);                      \
    }
EXL3_PREFILL_ENTRIES(1)
EXL3_PREFILL_ENTRIES(2)
EXL3_PREFILL_ENTRIES(3)
EXL3_PREFILL_ENTRIES(4)
EXL3_PREFILL_ENTRIES(5)
EXL3_PREFILL_ENTRIES(6)
EXL3_PREFILL_ENTRIES(7)
EXL3_PREFILL_ENTRIES(8)
