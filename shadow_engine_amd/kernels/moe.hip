// MoE glue for a verify batch: SwiGLU, the weighted combine, the fused router + group planner, exact top-64, and the
// greedy draft acceptance.  Semantics follow kernels/forward.cu of the reference (swiglu :2512, moe_combine_qwen_rows
// :2568, route_topk_rows :3169, route_plan_res_small :3392, topk_slices/_merge :3592-3630) and the accept loop of
// crates/shadowzero-serve/src/engine.rs:2377-2408.

// out = silu(g) * u over n values.
extern "C" __global__ void __launch_bounds__(256) swiglu(const float* g, const float* u, float* out, u32 n) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = siluf_ref(g[i]) * u[i];
}

// Token j = blockIdx.y: y[j] = sum over its cnt[j] experts t, in rank order, of w[j,t] * eo[j*k + t] + sigmoid(gl[j]) * sh_eo[j].
// sh_eo may be null (no shared expert).  grid = (ceil(n / 256), tokens).
extern "C" __global__ void __launch_bounds__(256) moe_combine_qwen_rows(float* y, const float* eo, const float* w, const float* sh_eo,
                                                                        const float* gl, const u32* cnt, u32 n, u32 k) {
    const u64 j = blockIdx.y;
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float* e = eo + j * k * n;
    const float* wj = w + j * k;
    if (k <= 16) {
        // every load goes out before the first is waited for (a loop over the count would take the count's round trip, then
        // one a rank); ranks past the count are read and not added
        float v[16], wt[16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            if ((u32) t < k) {
                v[t] = e[(u64) t * n + i];
                wt[t] = wj[t];
            }
        }
        const float sv = sh_eo ? sh_eo[j * n + i] : 0.0f;
        const float sg = sh_eo ? sigmoidf_ref(gl[j]) : 0.0f;
        const u32 c = cnt[j];
        float acc = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; t++)
            if ((u32) t < k && (u32) t < c) acc += wt[t] * v[t];
        if (sh_eo) acc += sg * sv;
        y[j * n + i] = acc;
        return;
    }
    float acc = 0.0f;
    const u32 c = cnt[j];
    for (u32 t = 0; t < c; t++) acc += wj[t] * e[(u64) t * n + i];
    if (sh_eo) acc += sigmoidf_ref(gl[j]) * sh_eo[j * n + i];
    y[j * n + i] = acc;
}

// ------------------------------------------------------------------------------------------------ router + planner
// Routing alone: tidx[j*k + t], weights[j*k + t] (f32), one wave a token.  grid = ceil(m / 4), block 256; ne <= 512, k <= 16.
// The weights are ex_t over the sum of the chosen ex (route_weights_chosen): a prefill chunk routes thousands of tokens, and
// the sum over all experts that cancels out of them is 512 f64 exponentials a token.
extern "C" __global__ void __launch_bounds__(256) route_topk_rows(const float* logits, u32* tidx, float* weights, u32 ne, u32 k, u32 m) {
    __shared__ double exs[4][512];
    __shared__ u32 tops[4][16];
    const u32 lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const u32 j = blockIdx.x * 4 + w;
    if (j >= m) return;
    route_ids(logits + (u64) j * ne, ne, k, lane, exs[w], tops[w]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    u32 count;
    const float wt = route_weights_chosen(logits + (u64) j * ne, ne, k, lane, tops[w], &count);
    if (lane < k) {
        tidx[(u64) j * k + lane] = tops[w][lane];
        weights[(u64) j * k + lane] = wt;
    }
}

// Fused router + group planner for a resident layer and a small batch: m <= 8 tokens, k <= 16, ne <= 512, G = m * k group
// slots per part.  One workgroup.  Writes into `base`, in the layout the grouped kernels read:
//   base + a0:         u64 addr[3][GT]   matrix address of every group: gate of every group, then up, then down
//   base + r0:         u32 rec[3][GT][17] {count, input rows[8], output rows[8]}; unused slots have count 0
//   base + w_off:      f32 weights[m][k]; base + counts_off: u32 cnt[m]; base + tidx_off: u32 tidx[m][k]
// with GT = G + nsh slots per part.  Pair (token j, rank t) is row j*k + t of the gate half and of the up half (up_off rows
// on) of the expert products, of act and of eo: gate and up read token j's row of the input, down reads the pair's row of
// act.  Tokens sharing an expert form one group (at most 4 tokens a group), groups in ascending expert order.  eaddr is
// the layer's table eaddr[part * ne + e] (crates/shadowzero-cuda/src/session.rs:2129-2146).  The nsh = ceil(m / 4) slots after the G routed ones
// carry the shared expert (address sh_addr[part], may be null: then they stay empty) for all m tokens: input row j,
// output row G + j (up: up_off + G + j).
extern "C" __global__ void __launch_bounds__(256) route_plan_res_small(const float* logits, const u64* eaddr, u8* base, u32 ne, u32 k, u32 m,
                                                                       u32 G, u32 up_off, u32 a0, u32 r0, u32 w_off, u32 counts_off,
                                                                       u32 tidx_off, const u64* sh_addr) {
    __shared__ double exs[4][512];
    __shared__ u32 tops[4][16];
    __shared__ u32 s_e[128];        // expert of pair p = j*k + t
    __shared__ u32 s_rank[128];     // position of the pair in (expert, token) order
    __shared__ u32 s_sorted[128];   // pair at each position
    __shared__ u32 s_head[128];     // 1 where a position starts a new group
    __shared__ u32 s_gid[128];      // group of each position
    const u32 tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const u32 N = m * k;
    const u32 nsh = (m + 3) / 4, GT = G + nsh;
    float* weights = (float*) (base + w_off);
    u32* cnt = (u32*) (base + counts_off);
    u32* tidx = (u32*) (base + tidx_off);
    for (u32 j = w; j < m; j += 4) {
        route_ids(logits + (u64) j * ne, ne, k, lane, exs[w], tops[w]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        u32 kk;
        const float wt = route_weights(logits + (u64) j * ne, ne, k, lane, tops[w], &kk);
        if (lane < k) {
            const u32 mine = tops[w][lane];
            s_e[j * k + lane] = mine;
            tidx[j * k + lane] = mine;
            weights[j * k + lane] = wt;
        }
        if (lane == 0) cnt[j] = kk;
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    // rank of every pair by (expert, pair index): a pair's token is j = p / k, so pair order is token order inside an expert
    if (tid < N) {
        const u32 e = s_e[tid];
        u32 r = 0;
        for (u32 p = 0; p < N; p++) {
            const u32 ep = s_e[p];
            r += (ep < e || (ep == e && p < tid)) ? 1u : 0u;
        }
        s_rank[tid] = r;
        s_sorted[r] = tid;
    }
    __syncthreads();
    if (tid < N) {
        // position tid: a group starts where the expert changes, or every 4th token of one expert
        const u32 p = s_sorted[tid], e = s_e[p];
        u32 first = tid;
        while (first > 0 && s_e[s_sorted[first - 1]] == e) first--;
        s_head[tid] = ((tid - first) % 4 == 0) ? 1u : 0u;
    }
    __syncthreads();
    if (tid < N) {
        u32 gsum = 0;
        for (u32 q = 0; q <= tid; q++) gsum += s_head[q];
        s_gid[tid] = gsum - 1;
    }
    __syncthreads();
    u64* addr = (u64*) (base + a0);
    u32* rec = (u32*) (base + r0);
    // clear every record's count first, then fill
    for (u32 i = tid; i < 3 * GT; i += 256) rec[(u64) i * 17] = 0u;
    __syncthreads();
    if (tid < N) {
        const u32 p = s_sorted[tid], e = s_e[p], g = s_gid[tid];
        if (e != 0xffffffffu) {
            u32 first = tid;
            while (s_head[first] == 0) first--;
            const u32 slot = tid - first;
            u32 len = 1;
            while (first + len < N && s_head[first + len] == 0) len++;
            const u32 j = p / k;
            for (u32 part = 0; part < 3; part++) {
                u32* r = rec + ((u64) part * GT + g) * 17;
                r[1 + slot] = part == 2 ? p : j;
                r[9 + slot] = part == 1 ? up_off + p : p;
                if (slot == 0) {
                    r[0] = len;
                    addr[(u64) part * GT + g] = eaddr[(u64) part * ne + e];
                }
            }
        }
    }
    if (sh_addr && tid < m) {
        const u32 g = G + tid / 4, slot = tid % 4;
        for (u32 part = 0; part < 3; part++) {
            u32* r = rec + ((u64) part * GT + g) * 17;
            r[1 + slot] = part == 2 ? G + tid : tid;
            r[9 + slot] = part == 1 ? up_off + G + tid : G + tid;
            if (slot == 0) {
                r[0] = min(4u, m - (tid / 4) * 4);
                addr[(u64) part * GT + g] = sh_addr[part];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------- exact top-64
// Order (tk_before of the reference, forward.cu:3560): value descending, then id ascending; a NaN counts as -inf, -0 equals +0.
// A candidate travels as one u64 key that orders exactly like that: the high word is the value's bit pattern made monotonic
// (-0 folded onto +0), the low word (0x7fffffff - id) * 2 + (1 if the value was -0), and 0 for a slot that holds nothing
// (value -inf, id 0xffffffff), so value and id come back out of the key bit for bit.
//
// A wave keeps its 64 best keys one a lane, sorted; compare-exchange steps are lane exchanges (DPP and lane swaps, no LDS, no
// barrier): a bitonic sort of 64 keys is 21 steps, and two sorted runs of opposite direction give their 64 best as the
// lane-wise larger key, a bitonic run that 6 more steps sort.  Which lanes keep the larger key of a step is a compile-time
// 64-bit constant, so a step is two lane moves, one 64-bit compare, a scalar xor of the compare's mask with the constant, and
// two selects.  (A 4096-key bitonic sort through LDS with a barrier a step, which this replaces, took 134 us a launch for
// the slices of four rows of a 151 936-word vocabulary; this takes a tenth.)
__device__ __forceinline__ u64 tk_key(float x, u32 id) {
    u32 b = f32_bits(x);
    if (x != x) b = 0xff800000u;
    const u32 negz = b == 0x80000000u ? 1u : 0u;
    if (negz) b = 0u;
    const u32 o = b ^ ((u32) ((i32) b >> 31) | 0x80000000u);
    const u32 lo = id == 0xffffffffu ? 0u : ((0x7fffffffu - id) << 1) | negz;
    return ((u64) o << 32) | lo;
}

__device__ __forceinline__ void tk_unkey(u64 k, float& x, u32& id) {
    const u32 o = (u32) (k >> 32), lo = (u32) k;
    u32 b = (o & 0x80000000u) ? o ^ 0x80000000u : ~o;
    if (lo & 1u) b = 0x80000000u;
    x = bits_f32(b);
    id = lo == 0u ? 0xffffffffu : 0x7fffffffu - (lo >> 1);
}

#define TK_NOTHING 0x007fffff00000000ull   /* tk_key(-inf, 0xffffffff) */

template <int J>
__device__ __forceinline__ u64 tk_partner(u64 k, u32 lane) {
    const u32 lo = f32_bits(lane_xor<J>(bits_f32((u32) k), lane)), hi = f32_bits(lane_xor<J>(bits_f32((u32) (k >> 32)), lane));
    return ((u64) hi << 32) | lo;
}

// The lanes that keep the larger key in step (K, J) of a bitonic sort of 64 lanes into descending (DESC) or ascending order:
// runs of K lanes alternate in direction, the lower lane of a pair J apart keeps the larger key in a descending run.
template <int K, int J, bool DESC>
constexpr u64 tk_keep_max() {
    u64 m = 0;
    for (int l = 0; l < 64; l++) {
        const bool main_dir = (l & K) == 0, lower = (l & J) == 0;
        if (DESC ? main_dir == lower : main_dir != lower) m |= 1ull << l;
    }
    return m;
}

template <int K, int J, bool DESC>
__device__ __forceinline__ void tk_step(u64& mine, u32 lane) {
    const u64 other = tk_partner<J>(mine, lane);
    constexpr u64 keep = tk_keep_max<K, J, DESC>();
    // where the larger key is kept the partner's is taken unless mine is larger; elsewhere it is taken if mine is larger
    const u64 take = __builtin_amdgcn_ballot_w64(mine > other) ^ keep;
#if __has_builtin(__builtin_amdgcn_inverse_ballot_w64)
    mine = __builtin_amdgcn_inverse_ballot_w64(take) ? other : mine;     // the mask selects as it stands: no vector work
#else
    mine = ((take >> lane) & 1) ? other : mine;                          // a compiler without it (an older run-time compiler) shifts
#endif
}

// Bitonic runs of K lanes -> sorted runs of K lanes (K = 64: the whole wave in the order DESC says).
template <int K, bool DESC>
__device__ __forceinline__ void tk_merge(u64& v, u32 lane) {
    if constexpr (K >= 64) tk_step<K, 32, DESC>(v, lane);
    if constexpr (K >= 32) tk_step<K, 16, DESC>(v, lane);
    if constexpr (K >= 16) tk_step<K, 8, DESC>(v, lane);
    if constexpr (K >= 8) tk_step<K, 4, DESC>(v, lane);
    if constexpr (K >= 4) tk_step<K, 2, DESC>(v, lane);
    tk_step<K, 1, DESC>(v, lane);
}

template <bool DESC>
__device__ __forceinline__ void tk_sort64(u64& v, u32 lane) {
    tk_merge<2, DESC>(v, lane);
    tk_merge<4, DESC>(v, lane);
    tk_merge<8, DESC>(v, lane);
    tk_merge<16, DESC>(v, lane);
    tk_merge<32, DESC>(v, lane);
    tk_merge<64, DESC>(v, lane);
}

__device__ __forceinline__ u64 tk_larger(u64 a, u64 b) { return a > b ? a : b; }

// The 64 best of up to 64 MAXCH keys by a workgroup of nw waves (a power of two; nw * PERW >= MAXCH): key(t) gives key t < n;
// 64-key chunks go to the waves in turn.  A wave sorts its chunks, alternately ascending and descending — independent
// chains of lane exchanges that fill each other's issue gaps — and halves their number level by level: the lane-wise larger
// key of an ascending and a descending run is a bitonic run of the 64 best of both, which 6 steps sort again.  The waves'
// runs are then halved in number through LDS until wave 0 holds the result (descending), which it returns.  sh holds 64
// keys a wave.
template <int MAXCH, int PERW, class F>
__device__ __forceinline__ u64 tk_best_of(u32 n, F key, u64* sh) {
    static_assert(PERW >= 2 && (PERW & (PERW - 1)) == 0, "a power of two");
    const u32 wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    u64 k[PERW];
#pragma unroll
    for (int c = 0; c < PERW; c++) {
        const u32 t = (c * nw + wave) * 64 + lane;
        k[c] = (c * nw < (u32) MAXCH && t < n) ? key(t) : TK_NOTHING;
    }
#pragma unroll
    for (int c = 0; c < PERW; c++) {
        if (c * nw < (u32) MAXCH && (c * nw + wave) * 64 < n) {     // uniform over the wave; a chunk of nothing is sorted as it is
            if (c & 1) tk_sort64<true>(k[c], lane);
            else tk_sort64<false>(k[c], lane);
        }
    }
#pragma unroll
    for (int w = 1; w < PERW; w *= 2) {
#pragma unroll
        for (int c = 0; c < PERW; c += 2 * w) {
            k[c] = tk_larger(k[c], k[c + w]);                        // ascending against descending
            if (2 * w == PERW || ((c / (2 * w)) & 1)) tk_merge<64, true>(k[c], lane);
            else tk_merge<64, false>(k[c], lane);
        }
    }
    u64 best = k[0];
    for (u32 half = nw >> 1; half > 0; half >>= 1) {
        if (wave >= half && wave < 2 * half) sh[wave * 64 + lane] = best;
        __syncthreads();
        if (wave < half) {
            best = tk_larger(best, sh[(wave + half) * 64 + 63 - lane]);     // the other run read backwards: ascending
            tk_merge<64, true>(best, lane);
        }
        __syncthreads();
    }
    return best;
}

// Up to 4096 keys by 16 waves (4 chunks a wave) or 4 waves (16 chunks a wave).
template <class F>
__device__ __forceinline__ u64 tk_best_of_4096(u32 n, F key, u64* sh) {
    return (blockDim.x >> 6) == 16 ? tk_best_of<64, 4>(n, key, sh) : tk_best_of<64, 16>(n, key, sh);
}

// Slice b of row r (blockIdx.x = r * nb + b): the 64 best of logits[r*stride + 4096 b .. +4096) into sv/si[(r*nb + b)*64 ..].
// Slots past the vocabulary hold (-inf, 0xffffffff).  grid = rows * nb, block 1024 or 256.
extern "C" __global__ void __launch_bounds__(1024) topk_slices(const float* logits, u32 vocab, u32 stride, u32 nb, float* sv, u32* si) {
    __shared__ u64 sh[1024];
    const u32 r = blockIdx.x / nb, b = blockIdx.x % nb;
    const float* row = logits + (u64) r * stride;
    const u32 first = b * 4096, n = vocab > first ? min(4096u, vocab - first) : 0u;
    const u64 best = tk_best_of_4096(n, [&](u32 t) { return tk_key(row[first + t], first + t); }, sh);
    if (threadIdx.x < 64) {
        float x;
        u32 id;
        tk_unkey(best, x, id);
        sv[(u64) blockIdx.x * 64 + threadIdx.x] = x;
        si[(u64) blockIdx.x * 64 + threadIdx.x] = id;
    }
}

// Row r = blockIdx.x: the 64 best of its nb * 64 slice winners (nb <= 64) into out[r*128 .. +64) (value bits) and
// out[r*128 + 64 .. +64) (ids).  grid = rows, block 1024 or 256.
extern "C" __global__ void __launch_bounds__(1024) topk_merge(const float* sv, const u32* si, u32 nb, u32* out) {
    __shared__ u64 sh[1024];
    const u32 r = blockIdx.x;
    const float* v = sv + (u64) r * nb * 64;
    const u32* id = si + (u64) r * nb * 64;
    const u64 best = tk_best_of_4096(min(nb * 64, 4096u), [&](u32 t) { return tk_key(v[t], id[t]); }, sh);
    if (threadIdx.x < 64) {
        float x;
        u32 i;
        tk_unkey(best, x, i);
        out[(u64) r * 128 + threadIdx.x] = f32_bits(x);
        out[(u64) r * 128 + 64 + threadIdx.x] = i;
    }
}

// ------------------------------------------------------------------------------------------ the 2-bit screen of the head
// The inexact, optional top-64 path of the reference (forward.cu:4371-4660; off unless asked for): the 2-bit copy of the head
// that exl3_build_q2_proxy_K made scores every output against the rows' int8 codes (proxy_q2_quant_x), the best score of a
// 128-output block is its mark, the k_blk best-marked blocks of every row are computed exactly (head_exl3_K with the list)
// and the top 64 are taken among those.
//
// Block ob = blockIdx.x, lane = output r of the block.  The score of r for row j: over the input blocks b in order,
// acc = fma(sh, fma(2 x_sc[j][b], sum_i code_i * u_i, x_corr[j][b]), acc) — the integer sums are dot-products-of-four of a
// code word with four levels (the level word shifted by 2 sl and masked gives inputs 4 sl' ..), exact in any order; the
// f32 part is the reference's, operation by operation.  The rows' codes are the same for every lane: they sit in LDS and
// are read as broadcasts, four words at a time.
// bmax[j * n_ob + ob] = the largest score of the block.  grid = out / 128, block 128.
template <int M>
__device__ __forceinline__ void proxy_q2_bmax(const u32* __restrict__ w_q2, const u16* __restrict__ w_sc, const u32* __restrict__ xq,
                                              const float* __restrict__ x_sc, const float* __restrict__ x_corr, float* __restrict__ bmax,
                                              u32 n_ob, u32 in_f, u32 m) {
    __shared__ __attribute__((aligned(16))) u32 s_xq[M][1024];      // the rows' codes: in <= 4096
    __shared__ float s_mx[2][M];
    const u32 ob = blockIdx.x, r = threadIdx.x, n_b = in_f / 128;
    for (u32 i = r; i < M * n_b * 32; i += 128) {
        const u32 j = i / (n_b * 32), k = i % (n_b * 32);
        s_xq[j][k] = j < m ? xq[(u64) j * n_b * 32 + k] : 0u;
    }
    __syncthreads();
    const u32x4* wq = (const u32x4*) w_q2 + (u64) ob * n_b * 256 + r;
    const u16* sc = w_sc + (u64) ob * n_b * 128 + r;
    float acc[M];
#pragma unroll
    for (int j = 0; j < M; j++) acc[j] = 0.0f;
#pragma unroll 2
    for (u32 b = 0; b < n_b; b++) {
        const u32x4 q[2] = {wq[(u64) b * 256], wq[(u64) b * 256 + 128]};
        const float wsc = f16_to_f32(sc[b * 128]);
        i32 ia[M];
#pragma unroll
        for (int j = 0; j < M; j++) ia[j] = 0;
#pragma unroll
        for (int hb = 0; hb < 2; hb++)
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                u32 u[4];
#pragma unroll
                for (int sl = 0; sl < 4; sl++) u[sl] = (q[hb][wi] >> (2 * sl)) & 0x03030303u;
#pragma unroll
                for (int j = 0; j < M; j++) {
                    const u32x4 xv = *(const u32x4*) &s_xq[j][b * 32 + hb * 16 + wi * 4];      // the same address in every lane
#pragma unroll
                    for (int sl = 0; sl < 4; sl++) ia[j] = __builtin_amdgcn_sdot4((i32) xv[sl], (i32) u[sl], ia[j], false);
                }
            }
#pragma unroll
        for (int j = 0; j < M; j++) {
            const u64 at = (u64) min((u32) j, m - 1) * n_b + b;
            acc[j] = __builtin_fmaf(wsc, __builtin_fmaf(2.0f * x_sc[at], (float) ia[j], x_corr[at]), acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < M; j++) {
        const float mx = wave_max_f32(acc[j]);
        if ((r & 63) == 0) s_mx[r >> 6][j] = mx;
    }
    __syncthreads();
    if (r < M && r < m) bmax[(u64) r * n_ob + ob] = fmaxf(s_mx[0][r], s_mx[1][r]);
}

extern "C" __global__ void __launch_bounds__(128) proxy_q2_bmax_m1(const u32* w_q2, const u16* w_sc, const u32* xq, const float* x_sc, const float* x_corr,
                                                                   float* bmax, u32 n_ob, u32 in_f, u32 m) {
    proxy_q2_bmax<1>(w_q2, w_sc, xq, x_sc, x_corr, bmax, n_ob, in_f, m);
}
extern "C" __global__ void __launch_bounds__(128) proxy_q2_bmax_m4(const u32* w_q2, const u16* w_sc, const u32* xq, const float* x_sc, const float* x_corr,
                                                                   float* bmax, u32 n_ob, u32 in_f, u32 m) {
    proxy_q2_bmax<4>(w_q2, w_sc, xq, x_sc, x_corr, bmax, n_ob, in_f, m);
}
extern "C" __global__ void __launch_bounds__(128) proxy_q2_bmax_m8(const u32* w_q2, const u16* w_sc, const u32* xq, const float* x_sc, const float* x_corr,
                                                                   float* bmax, u32 n_ob, u32 in_f, u32 m) {
    proxy_q2_bmax<8>(w_q2, w_sc, xq, x_sc, x_corr, bmax, n_ob, in_f, m);
}

// Row j = blockIdx.x: marks the k_blk best blocks of bmax[j][0 .. n_ob) in the bit map `seen` (forward.cu:4519-4563, with its
// way of choosing: thread t < 256 keeps the four best of blocks t, t + 256, .. — a strictly larger value replaces the fourth,
// so of equal values the earlier block stays; a NaN counts as -3e38 — and of the 1024 kept, ordered by value descending, block
// ascending, the first k_blk are marked; a thread that holds five of the k_blk best loses one, as there).  Only the set matters,
// so nothing is sorted across waves: each of the 16 waves sorts its 64 candidates and a candidate's place in the whole order
// is its place in its own run plus, by binary search, the number of better keys in the other 15.  grid = m, block 1024.
extern "C" __global__ void __launch_bounds__(1024) proxy_pick_rows(const float* bmax, u32 n_ob, u32 k_blk, u32* seen) {
    __shared__ u64 cand[1024];
    const u32 tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const float* row = bmax + (u64) blockIdx.x * n_ob;
    if (tid < 256) {
        // the thread's four best as sorted keys (value descending, block ascending, as the rest of the kernel orders them).  Its
        // blocks come in ascending order, so a key beats the fourth exactly when its value is strictly larger: of equal values
        // the earlier block stays, which is the reference's rule
        const u64 none = tk_key(-3.0e38f, 0xffffffffu);
        u64 best[4] = {none, none, none, none};
        for (u32 i = tid; i < n_ob; i += 256) {
            const float x = row[i];
            const u64 key = tk_key(x != x ? -3.0e38f : x, i);
            if (key > best[3]) {
                best[3] = key;
#pragma unroll
                for (int q = 3; q > 0; q--) {
                    const u64 hi = max(best[q - 1], best[q]), lo = min(best[q - 1], best[q]);
                    best[q - 1] = hi;
                    best[q] = lo;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) cand[tid * 4 + q] = best[q];
    }
    __syncthreads();
    u64 mine = cand[tid];
    tk_sort64<true>(mine, lane);
    __syncthreads();
    cand[tid] = mine;
    __syncthreads();
    u32 rank = lane;
#pragma unroll
    for (u32 w = 0; w < 16; w++) {
        const u64* run = cand + w * 64;       // descending
        u32 c = 0;                            // keys of the run that are better than mine
#pragma unroll
        for (u32 step = 32; step > 0; step >>= 1)
            if (run[c + step - 1] > mine) c += step;
        if (run[c] > mine) c++;
        if (w != wave) rank += c;
    }
    float x;
    u32 ob;
    tk_unkey(mine, x, ob);
    if (rank < k_blk && rank < n_ob && ob < n_ob) atomicOr(&seen[ob >> 5], 1u << (ob & 31));
}

// The marked blocks in ascending order into sel[1 ..], their number (at most max_sel; what does not fit is dropped) into
// sel[0]; the bit map is left cleared for the next call (forward.cu:4577-4622).  One wave: lane l takes words l, l + 64, ..
// grid 1, block 64.
extern "C" __global__ void __launch_bounds__(64) proxy_compact_seen(u32* seen, u32 n_ob, u32 max_sel, u32* sel) {
    const u32 lane = threadIdx.x, n_words = (n_ob + 31) >> 5;
    u32 base = 0;
    for (u32 w0 = 0; w0 < n_words; w0 += 64) {
        const u32 idx = w0 + lane;
        u32 mask = idx < n_words ? seen[idx] : 0u;
        if (idx < n_words) seen[idx] = 0u;
        const u32 cnt = __builtin_popcount(mask);
        // inclusive prefix sum of cnt over the lanes
        u32 pref = cnt;
        for (u32 off = 1; off < 64; off <<= 1) {
            const u32 o = (u32) __builtin_amdgcn_ds_bpermute((i32) ((lane - off) & 63) * 4, (i32) pref);
            if (lane >= off) pref += o;
        }
        u32 pos = base + pref - cnt;
        while (mask) {
            const u32 bit = (u32) __builtin_ctz(mask);
            mask &= mask - 1;
            if (pos < max_sel) sel[1 + pos] = idx * 32 + bit;
            pos++;
        }
        base += (u32) __builtin_amdgcn_readlane((i32) pref, 63);
    }
    if (lane == 0) sel[0] = min(base, max_sel);
}

// topk_slices over the packed logits of a block list (forward.cu:4626-4647): element i of row r (i < 128 sel[0]) is output
// sel[1 + i / 128] * 128 + i % 128; elements past the list hold (-inf, 0xffffffff).  The list ascends, so packed order is
// output order: candidates are ordered by their place and the place is turned into the output at the end.  grid = rows * nb,
// block 1024 or 256.
extern "C" __global__ void __launch_bounds__(1024) topk_slices_blks(const float* logits, u32 stride, const u32* sel, u32 nb, float* sv, u32* si) {
    __shared__ u64 sh[1024];
    const u32 r = blockIdx.x / nb, b = blockIdx.x % nb;
    const float* row = logits + (u64) r * stride;
    const u32 total = sel[0] << 7, first = b * 4096, n = total > first ? min(4096u, total - first) : 0u;
    const u64 best = tk_best_of_4096(n, [&](u32 t) { return tk_key(row[first + t], first + t); }, sh);
    if (threadIdx.x < 64) {
        float x;
        u32 at;
        tk_unkey(best, x, at);
        sv[(u64) blockIdx.x * 64 + threadIdx.x] = x;
        si[(u64) blockIdx.x * 64 + threadIdx.x] = at == 0xffffffffu ? at : (sel[1 + (at >> 7)] << 7) | (at & 127);
    }
}

// Greedy acceptance (engine.rs:2377-2408 without a sampler): ids[i] is the model's choice after batch row i; keep = 1 + the
// number of leading drafts d[i] that equal ids[i].  out[0] = keep, out[1] = the bonus token ids[keep - 1].  grid 1, block 64.
extern "C" __global__ void __launch_bounds__(64) verify_accept(const u32* ids, const u32* drafts, u32 n_drafts, u32* out) {
    // lane i compares draft i (n_drafts <= 63): the first lane that differs, or lane n_drafts, gives keep - 1; one round
    // trip to memory instead of one a draft
    const u32 i = threadIdx.x;
    const u32 a = ids[min(i, n_drafts)];
    const u32 d = i < n_drafts ? drafts[i] : 0u;
    const u64 stop = __builtin_amdgcn_ballot_w64(i >= n_drafts || a != d);
    const u32 first = (u32) __builtin_ctzll(stop);
    const u32 bonus = __builtin_amdgcn_readlane(a, first);
    if (i == 0) {
        out[0] = first + 1;
        out[1] = bonus;
    }
}

// A plain copy of n 16-byte words, grid-stride: the launch of known HBM traffic (16 n bytes read, 16 n written) against
// which the memory counters of a profile are scaled.
extern "C" __global__ void __launch_bounds__(256) copy_words16(const u32x4* src, u32x4* dst, u64 n) {
    const u64 step = (u64) gridDim.x * blockDim.x;
    for (u64 i = (u64) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) dst[i] = src[i];
}

// n bytes at p set to one value, grid-stride: the bytes up to the first 16-byte boundary and those past the last one go
// one a thread, the words between as 16-byte stores.  A kernel and not the runtime's memset, so that a caller may record
// it into a graph like any other launch.  grid = any, block 256.
extern "C" __global__ void __launch_bounds__(256) fill_bytes(u8* p, u32 byte, u64 n) {
    const u64 tid = (u64) blockIdx.x * blockDim.x + threadIdx.x, step = (u64) gridDim.x * blockDim.x;
    const u64 head = min(n, (u64) ((16 - ((u64) p & 15)) & 15)), words = (n - head) / 16, tail = n - head - 16 * words;
    const u32 b = byte & 0xffu, w = b * 0x01010101u;
    if (tid < head) p[tid] = (u8) b;
    if (tid < tail) p[head + 16 * words + tid] = (u8) b;
    u32x4* q = (u32x4*) (p + head);
    const u32x4 v = {w, w, w, w};
    for (u64 i = tid; i < words; i += step) q[i] = v;
}

// Staging a checkpoint: the pieces of one batch, copied to the device as one block, go to their places.  table[3 i ..] =
// (offset in src, offset in dst, bytes) of piece i; every piece is cut into 64 KiB units, unit blockIdx.x of piece
// blockIdx.y.  16-byte words when both addresses allow, else 4-byte words (EXL3 blobs are 4-byte aligned), else bytes.
// grid = (ceil(longest piece / 64 KiB), pieces), block 256.
extern "C" __global__ void __launch_bounds__(256) scatter_pieces(const u8* src, u8* dst, const u64* table, u32 n) {
    const u32 p = blockIdx.y;
    if (p >= n) return;
    const u64 so = table[3 * p], dof = table[3 * p + 1], len = table[3 * p + 2];
    const u64 lo = (u64) blockIdx.x << 16;
    if (lo >= len) return;
    const u64 cnt = min((u64) 65536, len - lo);
    const u8* s = src + so + lo;
    u8* d = dst + dof + lo;
    const u64 a = (u64) s | (u64) d;
    if ((a & 15) == 0) {
        const u32x4* s4 = (const u32x4*) s;
        u32x4* d4 = (u32x4*) d;
        for (u64 i = threadIdx.x; i < cnt / 16; i += 256) d4[i] = s4[i];
        for (u64 i = (cnt & ~15ull) + threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    } else if ((a & 3) == 0) {
        const u32* s1 = (const u32*) s;
        u32* d1 = (u32*) d;
        for (u64 i = threadIdx.x; i < cnt / 4; i += 256) d1[i] = s1[i];
        for (u64 i = (cnt & ~3ull) + threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    } else {
        for (u64 i = threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    }
}

// A snapshot of the recurrent state, or its restore: many device ranges copied by one launch (copy_many,
// kernels/forward.cu:3629; session.rs:3385-3404).  table[4 r ..] = (dst, src, bytes, first unit) of range r, the ranges cut
// into 64 KiB units that are numbered through (first unit of range r = units of the ranges before it): workgroup
// blockIdx.x takes unit blockIdx.x, whatever the sizes of the ranges, so a 2 MiB state and a 96 KiB one both fill the
// chip.  16-byte words when both addresses allow, else 4-byte words, else bytes.  grid = units of all ranges, block 256.
extern "C" __global__ void __launch_bounds__(256) copy_ranges(const u64* table, u32 n) {
    const u64 unit = blockIdx.x;
    u32 lo = 0, hi = n;                       // the last range whose first unit is <= unit
    while (hi - lo > 1) {
        const u32 mid = (lo + hi) / 2;
        if (table[4 * (u64) mid + 3] <= unit) lo = mid;
        else hi = mid;
    }
    const u64 len = table[4 * (u64) lo + 2];
    const u64 off = (unit - table[4 * (u64) lo + 3]) << 16;
    if (off >= len) return;
    const u64 cnt = min((u64) 65536, len - off);
    const u8* s = (const u8*) table[4 * (u64) lo + 1] + off;
    u8* d = (u8*) table[4 * (u64) lo] + off;
    const u64 a = (u64) s | (u64) d;
    if ((a & 15) == 0) {
        const u32x4* s4 = (const u32x4*) s;
        u32x4* d4 = (u32x4*) d;
        if (cnt == 65536) {
            // a whole unit: 16 words a thread, requested four at a time
#pragma unroll
            for (int r = 0; r < 4; r++) {
                u32x4 v[4];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = s4[threadIdx.x + 256 * (4 * r + i)];
#pragma unroll
                for (int i = 0; i < 4; i++) d4[threadIdx.x + 256 * (4 * r + i)] = v[i];
            }
            return;
        }
        for (u64 i = threadIdx.x; i < cnt / 16; i += 256) d4[i] = s4[i];
        for (u64 i = (cnt & ~15ull) + threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    } else if ((a & 3) == 0) {
        const u32* s1 = (const u32*) s;
        u32* d1 = (u32*) d;
        for (u64 i = threadIdx.x; i < cnt / 4; i += 256) d1[i] = s1[i];
        for (u64 i = (cnt & ~3ull) + threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    } else {
        for (u64 i = threadIdx.x; i < cnt; i += 256) d[i] = s[i];
    }
}

// ------------------------------------------------------------------------ the hyper-connection around a sublayer
// rmsnorm over every stream of every row on its own (forward.rs:251-260; rmsnorm_groups_rows of the reference): the mean
// of squares and the scaling in f64 as the CPU path has them, out = (float) (x * 1/sqrt(ms + eps)) * w.
// r, rn: [m][cs * h]; w: [cs * h].  grid = (cs, m), block 256.
extern "C" __global__ void __launch_bounds__(256) rmsnorm_groups_rows(const float* r, const float* w, float* rn, u32 h, float eps, u32 cs) {
    __shared__ double red[4];
    const u32 s = blockIdx.x, j = blockIdx.y, tid = threadIdx.x;
    const float* x = r + ((u64) j * cs + s) * h;
    double ss = 0.0;
    for (u32 i = tid; i < h; i += 256) ss += (double) x[i] * (double) x[i];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, SZ_WAVE);
    if (tid % 64 == 0) red[tid / 64] = ss;
    __syncthreads();
    const double ms = (((red[0] + red[1]) + red[2]) + red[3]) / (double) h;
    const double sc = 1.0 / sqrt(ms + (double) eps);
    float* o = rn + ((u64) j * cs + s) * h;
    for (u32 i = tid; i < h; i += 256) o[i] = (float) ((double) x[i] * sc) * w[s * h + i];
}

// u[j][i] = (sum over streams s, in order, of mix[j][s h + i] * rn[j][s h + i]) / cs (forward.rs:806-812; hc_mix_rows).
// grid = (ceil(h / 256), m), block 256.
extern "C" __global__ void __launch_bounds__(256) hc_mix_rows(const float* rn, const float* mix, float* u, u32 h, u32 cs) {
    const u32 i = blockIdx.x * 256 + threadIdx.x, j = blockIdx.y;
    if (i >= h) return;
    float a = 0.0f;
    for (u32 s = 0; s < cs; s++) a += mix[((u64) j * cs + s) * h + i] * rn[((u64) j * cs + s) * h + i];
    u[(u64) j * h + i] = a / (float) cs;
}

// hc_write (forward.rs:1078-1084): r[j][s h + i] += g[j][s] * y[j][i].  grid = (ceil(h / 256), cs, m), block 256.
extern "C" __global__ void __launch_bounds__(256) hc_write_rows(float* r, const float* g, const float* y, u32 h, u32 cs) {
    const u32 i = blockIdx.x * 256 + threadIdx.x, s = blockIdx.y, j = blockIdx.z;
    if (i >= h) return;
    float* o = r + ((u64) j * cs + s) * h + i;
    *o = *o + g[(u64) j * cs + s] * y[(u64) j * h + i];
}
