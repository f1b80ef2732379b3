// The prefill chunk of one MoE layer on int8 activations: tokens grouped by expert, IQ3_S weights decoded to signed int8
// in registers, int8 MFMA tiles (v_mfma_i32_16x16x32_i8: 16 tokens x 16 weight rows x one 32-weight sub-block), exact int32
// sub-block dots scaled by (weight scale x activation scale) in f32, SwiGLU, H re-quantized per 32, down into pair rows.
//
// Arithmetic follows the reference's CPU statement of the int8-activation expert (crates/shadowzero-model/src/cpu_expert.rs:99-110,
// 144-155, 217, 298-339 and cpu_expert_avx512.rs:25-42) with activation blocks of 32: d_x = amax / 127,
// q = clamp(round-half-away(v / d_x)); weights grid * sign as int8 with s_w = d (1 + 2 scale) per 32; a row's product is
// the sum over sub-blocks, in order, of (s_w * d_x) * (float) (int32 dot) in f32, each added with one fused multiply-add
// (the CPU statement rounds the product first: a last-bit difference now and then).  The launch structure is the
// native fused path's (native/fused/shadowzero_fused.cu:5-9: quantize, group, experts), re-made for wave64 MFMA.
//
// MFMA operand layout (16x16x32 i8): A (tokens x k) lane l holds row l % 16, k = 8 (l / 16) .. +8 as 8 bytes; B (k x rows)
// lane l holds column l % 16, the same k; C lane l holds column l % 16, rows 4 (l / 16) + r in acc[r].

//
// The ahead-of-time build has the matrix instructions write to ordinary vector registers: every tile's 4 sums a lane are
// converted and scaled at once, and out of the accumulation registers each would first cost a move (8 of 40 vector
// instructions a tile pair).
// hipcc: -mllvm -amdgpu-mfma-vgpr-form=1

typedef int i32x4 __attribute__((ext_vector_type(4)));

// q[i] = clamp(round(x[i] / d)), d[b] = amax / 127 over each 32 values (cpu_expert_avx512.rs:25-42).  One thread a block of 32.
__device__ __forceinline__ void quant_block_q8(const float* x, u64 b, i8* q, float* d) {
    const f32x4* p = (const f32x4*) (x + b * 32);
    float v[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 t = p[i];
        v[4 * i] = t.x;
        v[4 * i + 1] = t.y;
        v[4 * i + 2] = t.z;
        v[4 * i + 3] = t.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    const float dd = amax / 127.0f;
    const float id = dd > 0.0f ? 1.0f / dd : 0.0f;
    u32 w[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        u32 pack = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float r = fminf(127.0f, fmaxf(-127.0f, roundf(v[4 * i + k] * id)));
            pack |= ((u32) (int) r & 0xffu) << (8 * k);
        }
        w[i] = pack;
    }
    u32x4* o = (u32x4*) (q + b * 32);
    o[0] = u32x4{w[0], w[1], w[2], w[3]};
    o[1] = u32x4{w[4], w[5], w[6], w[7]};
    d[b] = dd;
}

// grid = ceil(n / 32 / 256), block 256.
extern "C" __global__ void __launch_bounds__(256) quant_act_q8(const float* x, u64 n, i8* q, float* d) {
    const u64 b = (u64) blockIdx.x * 256 + threadIdx.x;
    if (b < n / 32) quant_block_q8(x, b, q, d);
}

// The two things a chunk needs before its tokens can be grouped, in one launch (they do not depend on each other): the
// routing of its m tokens (workgroups [0, ceil(m / 4)): a wave a token, as route_topk_rows) and the quantization of its
// activations (the workgroups after them, as quant_act_q8).  grid = ceil(m / 4) + ceil(n / 32 / 256), block 256.
extern "C" __global__ void __launch_bounds__(256) prefill_front(const float* x, u64 n, i8* q, float* d, const float* logits, u32* tidx, float* weights,
                                                                u32 ne, u32 k, u32 m) {
    __shared__ double exs[4][512];
    __shared__ u32 tops[4][16];
    const u32 nr = (m + 3) / 4;
    if (blockIdx.x >= nr) {
        const u64 b = (u64) (blockIdx.x - nr) * 256 + threadIdx.x;
        if (b < n / 32) quant_block_q8(x, b, q, d);
        return;
    }
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

#define PF_TOK 64      // tokens of one work item: PF_TOK / 16 MFMA tiles of 16
#define PF_TILES (PF_TOK / 16)
#define PF_TOK_D 32    // tokens of one work item of the down kernel: with half the activations in LDS twice the workgroups fit a CU

// Groups the chunk's (token, rank) pairs by expert: offs[e] .. offs[e + 1] are the positions in list[] of expert e's pairs
// (pair = token * k + rank; the shared expert, index ne, takes the pairs npairs + token when nshared = tokens).  Also
// cnt[token] = its number of valid experts.  The order of an expert's pairs in list[] is arbitrary; every pair owns its
// output rows, so the results do not depend on it.  items[0] = the number of work items, items[1 + 2 i], items[2 + 2 i] =
// (expert, first position) of item i: every run of up to unit_gu pairs of an expert is one item of the gate/up kernel (at most
// ne + 1 + rows / unit_gu of them; PF_TOK for the int8 kernels below); items_d likewise with runs of up to unit_d pairs, for the down kernel.  The items that
// exist come first in both lists, so the workgroups launched for the rest of the bound run at the launches' ends, out of
// the way.  One workgroup.  grid 1, block 1024; ne <= 512.
extern "C" __global__ void __launch_bounds__(1024) prefill_group(const u32* tidx, u32 tokens, u32 k, u32 ne, u32 nshared, u32* offs, u32* list,
                                                                 u32* cnt, u32* items, u32* items_d, u32 unit_gu, u32 unit_d) {
    __shared__ u32 s_cnt[513], s_off[514], s_fill[513], s_fill_d[513];
    const u32 tid = threadIdx.x, npairs = tokens * k, nexp = ne + 1;
    for (u32 i = tid; i < nexp; i += 1024) {
        s_cnt[i] = 0;
        s_fill[i] = 0;
    }
    __syncthreads();
    for (u32 p = tid; p < npairs; p += 1024) {
        const u32 e = tidx[p];
        if (e < ne) atomicAdd(&s_cnt[e], 1u);
    }
    if (tid == 0) s_cnt[ne] = nshared;
    for (u32 j = tid; j < tokens; j += 1024) {
        u32 c = 0;
        for (u32 t = 0; t < k; t++) c += tidx[j * k + t] < ne ? 1u : 0u;
        cnt[j] = c;
    }
    __syncthreads();
    // three running sums over the experts, each by a wave of its own: lane L takes the experts [9 L, 9 L + 9) (ne <= 512), the
    // lanes' totals are scanned across the wave, and every lane writes its experts' starts
    {
        const u32 w = tid >> 6, lane = tid & 63;
        if (w < 3) {
            const u32 unit = w == 0 ? 1u : w == 1 ? unit_gu : unit_d;   // pairs; gate/up items; down items
            u32 v[9], sum = 0;
#pragma unroll
            for (int q = 0; q < 9; q++) {
                const u32 i = 9 * lane + q;
                v[q] = i < nexp ? (s_cnt[i] + unit - 1) / unit : 0u;
                sum += v[q];
            }
            u32 incl = sum;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const u32 up = __shfl_up(incl, o, SZ_WAVE);
                if (lane >= (u32) o) incl += up;
            }
            u32 run = incl - sum;
            u32* dst = w == 0 ? s_off : w == 1 ? s_fill : s_fill_d;   // s_fill is borrowed until the barrier below; it is cleared again before the fill
#pragma unroll
            for (int q = 0; q < 9; q++) {
                const u32 i = 9 * lane + q;
                if (i < nexp) dst[i] = run;
                run += v[q];
            }
            if (lane == 63) {
                if (w == 0) s_off[nexp] = incl;
                else if (w == 1) items[0] = incl;
                else items_d[0] = incl;
            }
        }
    }
    __syncthreads();
    for (u32 i = tid; i < nexp; i += 1024) {
        u32 ni = s_fill[i];
        for (u32 t0 = 0; t0 < s_cnt[i]; t0 += unit_gu, ni++) {
            items[1 + 2 * ni] = i;
            items[2 + 2 * ni] = t0;
        }
        ni = s_fill_d[i];
        for (u32 t0 = 0; t0 < s_cnt[i]; t0 += unit_d, ni++) {
            items_d[1 + 2 * ni] = i;
            items_d[2 + 2 * ni] = t0;
        }
    }
    __syncthreads();
    for (u32 i = tid; i < nexp; i += 1024) s_fill[i] = 0;
    __syncthreads();
    for (u32 i = tid; i <= nexp; i += 1024) offs[i] = s_off[i];
    for (u32 p = tid; p < npairs; p += 1024) {
        const u32 e = tidx[p];
        if (e < ne) list[s_off[e] + atomicAdd(&s_fill[e], 1u)] = p;
    }
    for (u32 j = tid; j < nshared; j += 1024) list[s_off[ne] + j] = npairs + j;
}

__shared__ u32 pf_grid[512];
__shared__ u64 pf_sign[256];   // a sign byte as eight byte masks: 0xff where the bit is set

// Fills the two tables; every thread of the workgroup (256) calls it, and a barrier must follow before they are read.
__device__ __forceinline__ void pf_tables(u32 tid) {
    for (u32 i = tid; i < 512; i += 256) pf_grid[i] = IQ3S_GRID[i];
    u64 m = 0;
#pragma unroll
    for (int b = 0; b < 8; b++) m |= ((tid >> b) & 1u) ? (0xffull << (8 * b)) : 0ull;
    pf_sign[tid] = m;
}

// Eight consecutive weights (k = 8 kq .. 8 kq + 7 of sub-block g) of one IQ3_S block at `blk` (LDS, 2-byte aligned) as
// signed int8 (cpu_expert.rs:99-110).
__device__ __forceinline__ u64 iq3s_int8x8(const u8* blk, u32 g, u32 kq) {
    const u32 j = 8 * g + 2 * kq;                       // index of the first of the two 4-weight groups
    const u32 qs = *(const u16*) (blk + 2 + j);
    const u32 qh = blk[66 + g] >> (2 * kq);
    const u32 signs = blk[74 + 4 * g + kq];
    const u32 g0 = pf_grid[(qs & 0xff) | ((qh & 1u) << 8)], g1 = pf_grid[(qs >> 8) | ((qh & 2u) << 7)];
    // negate the bytes whose sign bit is set: (m ^ mask) + (mask & 1) per byte, magnitudes are at most 15 so nothing carries
    const u64 mask = pf_sign[signs];
    const u32 m0 = (u32) mask, m1 = (u32) (mask >> 32);
    const u32 w0 = (g0 ^ m0) + (m0 & 0x01010101u), w1 = (g1 ^ m1) + (m1 & 0x01010101u);
    return ((u64) w1 << 32) | w0;
}

// The sub-block scales d (1 + 2 s) of a block: the four lanes that share a row (kq = 0..3) would each work out all eight;
// instead lane (n, kq) works out the two of the byte it is handed (sub-blocks 2 kq and 2 kq + 1) and leaves them in the wave's
// own strip sw[8][16] (LDS), where the products read them back (a quarter of the arithmetic, conflict-free reads).
// A wavefront fence must follow before the strip is read.
__device__ __forceinline__ void iq3s_scales_to_strip(const u8* blk, u32 n, u32 kq, float* sw) {
    const float d = f16_to_f32(*(const u16*) blk);
    const u32 sc = blk[106 + kq];
    sw[(2 * kq) * 16 + n] = d * (float) (1 + 2 * (sc & 0x0f));
    sw[(2 * kq + 1) * 16 + n] = d * (float) (1 + 2 * (sc >> 4));
}

#define PF_KC 256      // k of one staged chunk: one IQ3_S block a row
#define PF_AB(TOK) ((TOK) * 256)   // a chunk's activations in LDS: [tokens][16 columns of 16 bytes], column c of token t at slot c ^ (t & 15)
#define PF_DB(TOK) ((TOK) * 32)    // a chunk's activation scales in LDS: [8 sub-blocks][tokens]
#define PF_WB 7168     // a chunk's 64 blocks of one matrix in LDS: 28 words a row
#define PF_WS 112      // bytes between rows there

// A chunk is brought into LDS by global-to-LDS loads (no registers in between), every wave a quarter of them, one chunk
// ahead of the products: while the matrix and vector units work on chunk c the loads of chunk c + 1 are in flight into the
// other buffer.  A wave's load instruction fills 64 consecutive slots of LDS from 64 addresses of its choosing, so the
// layout is made by choosing the addresses.

// The int8 activations and their scales of TOK pairs (32 or 64) for k in [k0, k0 + 256).  Token t's 16-byte column c lands at
// slot c ^ (t & 15) of its row: the 16 tokens of an MFMA tile then read the same column from 16 different bank groups.
// `rows` (LDS): the row of q and d every pair reads; a pair past the item's end names row 0, whose products are dropped.
template <int TOK, int NWV = 4>   // NWV: the waves that share the chunk's loads
__device__ __forceinline__ void pf_issue_a(const i8* __restrict__ q, const float* __restrict__ d, const u32* rows, u32 cols, u32 k0, u32 lds_a,
                                           u32 lds_d, u32 wave, u32 lane) {
    static_assert((TOK / 8) % NWV == 0, "every wave the same number of load instructions");
#pragma unroll
    for (int it = 0; it < TOK / 4 / NWV; it++) {          // TOK / 4 instructions a chunk: 4 tokens each
        const u32 j = wave * (TOK / 4 / NWV) + it, t = 4 * j + (lane >> 4), c = (lane & 15) ^ (t & 15);
        lds_load<16>(q + (u64) rows[t] * cols + k0 + 16 * c, lds_a + j * 1024);
    }
#pragma unroll
    for (int it = 0; it < TOK / 8 / NWV; it++) {          // TOK / 8 instructions: 64 of the 8 x TOK scales each
        const u32 j = wave * (TOK / 8 / NWV) + it, i = j * 64 + lane, g = i / TOK, t = i % TOK;
        lds_load<4>(d + (u64) rows[t] * (cols / 32) + k0 / 32 + g, lds_d + j * 256);
    }
}

// Block `c` (the 256 weights k in [256 c, 256 c + 256)) of 64 consecutive rows of a row-major IQ3_S matrix: 28 words a
// row.  Blocks are only 2-byte aligned: a row's words start at the word that holds the block's first byte, and the block
// begins pf_shift (0 or 2) bytes into its slot.  The words of a row never leave the matrix: its first block starts on a
// word and its last one ends on one (a row is a multiple of 4 bytes, or rows come in even numbers).
// w = the first of the 64 rows, rb = bytes a row.
__device__ __forceinline__ u32 pf_shift(const u8* w, u32 rb, u32 c, u32 row) { return (u32) ((u64) (w + (u64) row * rb + c * 110) & 2); }
template <int NWV = 4>
__device__ __forceinline__ void pf_issue_w(const u8* __restrict__ w, u32 rb, u32 c, u32 lds_w, u32 wave, u32 lane) {
#pragma unroll
    for (int it = 0; it < (28 + NWV - 1) / NWV; it++) {   // 28 instructions a chunk and matrix: 64 rows x 28 words
        const u32 j = NWV == 4 ? wave * 7 + it : wave + NWV * it;
        if (j < 28) {                                     // (wave-uniform)
            const u32 i = j * 64 + lane, row = i / 28, dw = i % 28;
            const u8* a = w + (u64) row * rb + c * 110;
            lds_load<4>(a - ((u64) a & 2) + 4 * dw, lds_w + j * 256);
        }
    }
}

// One staged chunk's products: for each of its 8 sub-blocks the lane's 8 weights of its row (gate and up, or down) against
// the first T token tiles, every tile's exact int32 sums scaled and added in f32 (a fused multiply-add a sum, in sub-block
// order).  aq, ad: the chunk's activations and their scales; bg, bu, bd: the lane's row's block in LDS.
template <int V> struct pf_int { static constexpr int value = V; };

// NG sub-blocks from G0 on (8 from 0: the whole block; 4 from 0 or 4: a wave's half where two waves share a row group).
template <int T, int TOK, int NG = 8, int G0 = 0>
__device__ __forceinline__ void pf_products_gu(float (&accg)[PF_TILES][4], float (&accu)[PF_TILES][4], const u8* aq, const float* ad, const u8* bg, const u8* bu,
                                               u32 n, u32 kq, float* sw) {
    constexpr u32 g0 = G0;
    iq3s_scales_to_strip(bg, n, kq, sw);
    iq3s_scales_to_strip(bu, n, kq, sw + 128);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (u32 gg = 0; gg < NG; gg++) {
        const u32 g = g0 + gg;
        const float swg = sw[g * 16 + n], swu = sw[128 + g * 16 + n];
        const u64 b_g = iq3s_int8x8(bg, g, kq), b_u = iq3s_int8x8(bu, g, kq);
        const u32 col = ((2 * g + (kq >> 1)) ^ n) * 16 + 8 * (kq & 1);   // where this lane's 8 activations of a token lie in its row
#pragma unroll
        for (int a = 0; a < T; a++) {
            const u64 av = *(const u64*) (aq + (16 * a + n) * 256 + col);
            const f32x4 dx = *(const f32x4*) (ad + g * TOK + 16 * a + 4 * kq);
            const i32x4 z = {0, 0, 0, 0};
            const i32x4 cg = __builtin_amdgcn_mfma_i32_16x16x32_i8((long) av, (long) b_g, z, 0, 0, 0);
            const i32x4 cu = __builtin_amdgcn_mfma_i32_16x16x32_i8((long) av, (long) b_u, z, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                accg[a][r] = __builtin_fmaf(swg * dx[r], (float) cg[r], accg[a][r]);
                accu[a][r] = __builtin_fmaf(swu * dx[r], (float) cu[r], accu[a][r]);
            }
        }
    }
}
template <int T, int TOK>
__device__ __forceinline__ void pf_products_d(float (&acc)[TOK / 16][4], const u8* aq, const float* ad, const u8* bd, u32 n, u32 kq, float* sws) {
    iq3s_scales_to_strip(bd, n, kq, sws);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (u32 g = 0; g < 8; g++) {
        const float sw = sws[g * 16 + n];
        const u64 b = iq3s_int8x8(bd, g, kq);
        const u32 col = ((2 * g + (kq >> 1)) ^ n) * 16 + 8 * (kq & 1);
#pragma unroll
        for (int a = 0; a < T; a++) {
            const u64 av = *(const u64*) (aq + (16 * a + n) * 256 + col);
            const f32x4 dx = *(const f32x4*) (ad + g * TOK + 16 * a + 4 * kq);
            const i32x4 z = {0, 0, 0, 0};
            const i32x4 cc = __builtin_amdgcn_mfma_i32_16x16x32_i8((long) av, (long) b, z, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[a][r] = __builtin_fmaf(sw * dx[r], (float) cc[r], acc[a][r]);
        }
    }
}

// Work item blockIdx.y = (expert, first position) from prefill_group: gate and up rows [64 blockIdx.x + 16 (wave & 3), +16) of
// the expert against up to 64 of its pairs' tokens, SwiGLU (silu in f32, cpu_expert.rs:217), and H re-quantized per 32
// features: hq[pair][ff], hd[pair][ff / 32].  eaddr[part * ne + e] / sh_addr[part] as in the planner's kernels.
// grid = (ff / 64, the bound on the number of items), block 64 NWV.
// NWV = 4: wave w rows 16 w .. 16 w + 15, all 8 sub-blocks of a chunk's block.  NWV = 8 (block 512): waves w and w + 4 share
// the rows 16 (w & 3) .. and take sub-blocks 0..3 and 4..7 of every block; their partial sums are added at the end (the same
// LDS a workgroup, twice the waves a SIMD to cover the LDS reads and the barriers of a chunk).
template <int NWV>
__device__ __forceinline__ void prefill_gate_up_iq3_s_body(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list, const u32* items,
                                                           const i8* xq, const float* xd, i8* hq, float* hd, u32 ne, u32 k, u32 npairs, u32 hidden, u32 ff) {
    // two buffers of a chunk: activations | gate rows | up rows | activation scales; afterwards the item's 64 x 64 block of H
    constexpr u32 AB = PF_AB(PF_TOK), BUF = AB + 2 * PF_WB + PF_DB(PF_TOK);
    __shared__ __attribute__((aligned(16))) u8 stage[2 * BUF];
    __shared__ u32 s_rows[PF_TOK], s_pairs[PF_TOK];
    __shared__ float s_sw[NWV][256];   // a wave's strip of sub-block scales: gate [8][16], up [8][16]
    static_assert(sizeof(stage) >= 3 * PF_TOK * 65 * sizeof(float), "H and the second half's partial sums reuse the staging area");
    float (*hs)[65] = (float (*)[65]) stage;
    const u32 tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const u32 n = lane & 15, kq = lane >> 4;
    const u32 rw = wave & 3, kh = wave >> 2;             // the wave's row group; which half of the sub-blocks (NWV = 8)
    const u32 lrow = rw * 16 + n;                        // the lane's weight row inside the workgroup's 64
    const u32 rb = hidden / 256 * 110, rbx = blockIdx.x;
    const u32 lds0 = __builtin_amdgcn_readfirstlane(lds_offset(stage));
    if (blockIdx.y >= items[0]) return;
    const u32 e = items[1 + 2 * blockIdx.y], t0 = items[2 + 2 * blockIdx.y];
    if (e == ne && !sh_addr) return;
    const u32 first = offs[e], nt = min((u32) PF_TOK, offs[e + 1] - first - t0);
    if (tid < 256) pf_tables(tid);
    const u8* wg = (const u8*) (e < ne ? eaddr[e] : sh_addr[0]) + (u64) rbx * 64 * rb;
    const u8* wu = (const u8*) (e < ne ? eaddr[(u64) ne + e] : sh_addr[1]) + (u64) rbx * 64 * rb;
    if (tid < PF_TOK) {
        const u32 p = tid < nt ? list[first + t0 + tid] : 0;
        s_pairs[tid] = p;
        s_rows[tid] = p < npairs ? p / k : p - npairs;
    }
    float accg[PF_TILES][4], accu[PF_TILES][4];
#pragma unroll
    for (int a = 0; a < PF_TILES; a++)
#pragma unroll
        for (int r = 0; r < 4; r++) accg[a][r] = accu[a][r] = 0.0f;
    __syncthreads();   // s_rows and the tables are written
    auto issue = [&](u32 c) {
        const u32 base = lds0 + (c & 1) * BUF;
        pf_issue_a<PF_TOK, NWV>(xq, xd, s_rows, hidden, c * PF_KC, base, base + AB + 2 * PF_WB, wave, lane);
        pf_issue_w<NWV>(wg, rb, c, base + AB, wave, lane);
        pf_issue_w<NWV>(wu, rb, c, base + AB + PF_WB, wave, lane);
    };
    const u32 nc = hidden / PF_KC;
    constexpr int NG = NWV == 8 ? 4 : 8;
    // The loop over the chunks, straight-line code for the item's number of token tiles T (the scheduler overlaps one tile's
    // loads and matrix instructions with the scaling of the tile before it) and, with 8 waves, for the wave's half of the
    // sub-blocks: chosen once, outside the loop, so that only T tiles' sums are live in it.
    auto chunks = [&](auto tiles, auto half) {
        constexpr int T = decltype(tiles)::value, G0 = decltype(half)::value;
        float ag[PF_TILES][4], au[PF_TILES][4];
#pragma unroll
        for (int a = 0; a < T; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) ag[a][r] = au[a][r] = 0.0f;
        issue(0);
        for (u32 c = 0; c < nc; c++) {
            wait_vm<0>();
            __syncthreads();   // chunk c is in LDS, from every wave; the products of chunk c - 1 are done, so its buffer is free
            if (c + 1 < nc) issue(c + 1);
            const u8* buf = stage + (c & 1) * BUF;
            const u8* aq = buf;
            const float* ad = (const float*) (buf + AB + 2 * PF_WB);
            const u8* bg = buf + AB + lrow * PF_WS + pf_shift(wg, rb, c, lrow);
            const u8* bu = buf + AB + PF_WB + lrow * PF_WS + pf_shift(wu, rb, c, lrow);
            pf_products_gu<T, PF_TOK, NG, G0>(ag, au, aq, ad, bg, bu, n, kq, s_sw[wave]);
        }
#pragma unroll
        for (int a = 0; a < T; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                accg[a][r] = ag[a][r];
                accu[a][r] = au[a][r];
            }
    };
    auto halves = [&](auto tiles) {
        if (NWV == 8 && kh == 1) chunks(tiles, pf_int<4>{});
        else chunks(tiles, pf_int<0>{});
    };
    switch ((nt + 15) / 16) {
        case 1: halves(pf_int<1>{}); break;
#if PF_TILES > 2
        case 2: halves(pf_int<2>{}); break;
        case 3: halves(pf_int<3>{}); break;
#endif
        default: halves(pf_int<PF_TILES>{}); break;
    }
    __syncthreads();   // the staging area becomes H
    if constexpr (NWV == 8) {
        // the second half's partial sums go through LDS to the wave that holds the first half's
        float (*pg)[65] = (float (*)[65]) (stage + PF_TOK * 65 * sizeof(float));
        float (*pu)[65] = (float (*)[65]) (stage + 2 * PF_TOK * 65 * sizeof(float));
        if (kh == 1) {
#pragma unroll
            for (int a = 0; a < PF_TILES; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    pg[16 * a + 4 * kq + r][16 * rw + n] = accg[a][r];
                    pu[16 * a + 4 * kq + r][16 * rw + n] = accu[a][r];
                }
        }
        __syncthreads();
        if (kh == 0) {
#pragma unroll
            for (int a = 0; a < PF_TILES; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    accg[a][r] += pg[16 * a + 4 * kq + r][16 * rw + n];
                    accu[a][r] += pu[16 * a + 4 * kq + r][16 * rw + n];
                }
        }
    }
    // H = silu(gate) * up for (token 16 a + 4 kq + r, feature 16 rw + n), then per-32 quantization over features
    if (kh == 0) {
#pragma unroll
        for (int a = 0; a < PF_TILES; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) hs[16 * a + 4 * kq + r][16 * rw + n] = (accg[a][r] / (1.0f + expf(-accg[a][r]))) * accu[a][r];
    }
    __syncthreads();
    if (tid < 2 * PF_TOK) {
        const u32 t = tid >> 1, half = tid & 1;
        if (t < nt) {
            float amax = 0.0f;
            for (u32 i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(hs[t][32 * half + i]));
            const float dd = amax / 127.0f;
            const float id = dd > 0.0f ? 1.0f / dd : 0.0f;
            const u32 p = s_pairs[t];
            i8* o = hq + (u64) p * ff + rbx * 64 + 32 * half;
            for (u32 i = 0; i < 32; i++) o[i] = (i8) (int) fminf(127.0f, fmaxf(-127.0f, roundf(hs[t][32 * half + i] * id)));
            hd[(u64) p * (ff / 32) + rbx * 2 + half] = dd;
        }
    }
}

extern "C" __global__ void __launch_bounds__(512, 4) prefill_gate_up_iq3_s(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list,
                                                                        const u32* items, const i8* xq, const float* xd, i8* hq, float* hd, u32 ne,
                                                                        u32 k, u32 npairs, u32 hidden, u32 ff) {
    prefill_gate_up_iq3_s_body<8>(eaddr, sh_addr, offs, list, items, xq, xd, hq, hd, ne, k, npairs, hidden, ff);
}
// The same with four waves a workgroup (block 256), every wave the whole of its rows' blocks: kept for comparisons.
extern "C" __global__ void __launch_bounds__(256, 2) prefill_gate_up_iq3_s_w4(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list,
                                                                           const u32* items, const i8* xq, const float* xd, i8* hq, float* hd, u32 ne,
                                                                           u32 k, u32 npairs, u32 hidden, u32 ff) {
    prefill_gate_up_iq3_s_body<4>(eaddr, sh_addr, offs, list, items, xq, xd, hq, hd, ne, k, npairs, hidden, ff);
}

// Work item blockIdx.y: down rows of the expert against its pairs' H: eo[pair][hidden], unweighted (cpu_expert.rs:316-339).
// A workgroup takes hidden / 64 / gridDim.x blocks of 64 rows one after the other (wave w rows 16 w .. 16 w + 15 of each):
// its set-up is paid once, and the loads of a block's first chunk are in flight while the block before it is multiplied.
// items: prefill_group's list of runs of up to PF_TOK_D pairs.
// grid = (a divisor of hidden / 64, the bound on the number of those items), block 256.
extern "C" __global__ void __launch_bounds__(256, 4) prefill_down_iq3_s(const u64* eaddr, const u64* sh_addr, const u32* offs, const u32* list,
                                                                     const u32* items, const i8* hq, const float* hd, float* eo, u32 ne, u32 hidden,
                                                                     u32 ff) {
    constexpr u32 TOK = PF_TOK_D, AB = PF_AB(TOK), BUF = AB + PF_WB + PF_DB(TOK);   // two buffers of a chunk: activations | rows | activation scales
    __shared__ __attribute__((aligned(16))) u8 stage[2 * BUF];
    __shared__ u32 s_pairs[TOK];
    __shared__ float s_sw[4][128];   // a wave's strip of sub-block scales [8][16]
    const u32 tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const u32 n = lane & 15, kq = lane >> 4;
    const u32 lrow = wave * 16 + n;
    const u32 rb = ff / 256 * 110;
    const u32 per = hidden / 64 / gridDim.x, rb0 = blockIdx.x * per;     // this workgroup's row blocks: rb0 .. rb0 + per - 1
    const u32 lds0 = __builtin_amdgcn_readfirstlane(lds_offset(stage));
    if (blockIdx.y >= items[0]) return;
    const u32 e = items[1 + 2 * blockIdx.y], t0 = items[2 + 2 * blockIdx.y];
    if (e == ne && !sh_addr) return;
    const u32 first = offs[e], nt = min((u32) TOK, offs[e + 1] - first - t0);
    pf_tables(tid);
    const u8* wd = (const u8*) (e < ne ? eaddr[2ull * ne + e] : sh_addr[2]) + (u64) rb0 * 64 * rb;
    if (tid < TOK) s_pairs[tid] = tid < nt ? list[first + t0 + tid] : 0;
    float acc[TOK / 16][4];
#pragma unroll
    for (int a = 0; a < TOK / 16; a++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[a][r] = 0.0f;
    __syncthreads();   // s_pairs and the tables are written
    const u32 nc = ff / PF_KC, units = per * nc;   // a unit: one chunk of one row block
    auto issue = [&](u32 u) {
        const u32 base = lds0 + (u & 1) * BUF, c = u % nc;
        pf_issue_a<TOK>(hq, hd, s_pairs, ff, c * PF_KC, base, base + AB + PF_WB, wave, lane);
        pf_issue_w(wd + (u64) (u / nc) * 64 * rb, rb, c, base + AB, wave, lane);
    };
    issue(0);
    for (u32 u = 0; u < units; u++) {
        wait_vm<0>();
        __syncthreads();   // unit u is in LDS, from every wave; the products of unit u - 1 are done, so its buffer is free
        if (u + 1 < units) issue(u + 1);
        const u32 c = u % nc, rbi = u / nc;
        const u8* buf = stage + (u & 1) * BUF;
        const u8* aq = buf;
        const float* ad = (const float*) (buf + AB + PF_WB);
        const u8* bd = buf + AB + lrow * PF_WS + pf_shift(wd + (u64) rbi * 64 * rb, rb, c, lrow);
        if (nt <= 16) pf_products_d<1, TOK>(acc, aq, ad, bd, n, kq, s_sw[wave]);
        else pf_products_d<2, TOK>(acc, aq, ad, bd, n, kq, s_sw[wave]);
        if (c + 1 == nc) {   // the row block is complete
            const u32 row = (rb0 + rbi) * 64 + lrow;
#pragma unroll
            for (int a = 0; a < TOK / 16; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const u32 t = 16 * a + 4 * kq + r;
                    if (t < nt) eo[(u64) s_pairs[t] * hidden + row] = acc[a][r];
                    acc[a][r] = 0.0f;
                }
        }
    }
}
