// Wave-level routing helpers shared by the MoE glue kernels and the fused EXL3 verify kernels.
// Wave-wide reductions over DPP row shifts and broadcasts (no LDS round trips): after the six steps lane 63 holds the
// result, which readlane hands to every lane.
#define SZ_DPP(v, ctrl, rmask) __builtin_amdgcn_update_dpp((v), (v), (ctrl), (rmask), 0xf, false)

__device__ __forceinline__ u64 wave_max_u64(u64 v) {
#define SZ_STEP(ctrl, rmask)                                                                \
    {                                                                                       \
        const u32 lo = SZ_DPP((u32) v, ctrl, rmask), hi = SZ_DPP((u32) (v >> 32), ctrl, rmask); \
        const u64 o = ((u64) hi << 32) | lo;                                                \
        v = o > v ? o : v;                                                                  \
    }
    SZ_STEP(0xb1, 0xf)    // quad_perm [1,0,3,2]
    SZ_STEP(0x4e, 0xf)    // quad_perm [2,3,0,1]
    SZ_STEP(0x114, 0xf)   // row_shr:4
    SZ_STEP(0x118, 0xf)   // row_shr:8
    SZ_STEP(0x142, 0xa)   // row_bcast:15 into rows 1 and 3
    SZ_STEP(0x143, 0xc)   // row_bcast:31 into rows 2 and 3
#undef SZ_STEP
    const u32 lo = __builtin_amdgcn_readlane((u32) v, 63), hi = __builtin_amdgcn_readlane((u32) (v >> 32), 63);
    return ((u64) hi << 32) | lo;
}

__device__ __forceinline__ u32 wave_min_u32(u32 v) {
    v = min(v, (u32) SZ_DPP(v, 0xb1, 0xf));
    v = min(v, (u32) SZ_DPP(v, 0x4e, 0xf));
    v = min(v, (u32) SZ_DPP(v, 0x114, 0xf));
    v = min(v, (u32) SZ_DPP(v, 0x118, 0xf));
    v = min(v, (u32) SZ_DPP(v, 0x142, 0xa));
    v = min(v, (u32) SZ_DPP(v, 0x143, 0xc));
    return __builtin_amdgcn_readlane(v, 63);
}

__device__ __forceinline__ float wave_max_f32(float v) {
#define SZ_STEP(ctrl, rmask) v = fmaxf(v, bits_f32(SZ_DPP(f32_bits(v), ctrl, rmask)));
    SZ_STEP(0xb1, 0xf) SZ_STEP(0x4e, 0xf) SZ_STEP(0x114, 0xf) SZ_STEP(0x118, 0xf) SZ_STEP(0x142, 0xa) SZ_STEP(0x143, 0xc)
#undef SZ_STEP
    return bits_f32(__builtin_amdgcn_readlane(f32_bits(v), 63));
}

// forward::route (forward.rs:1088) for one token by one wave, exactly: f32 maximum, exp of (logit - max) in f64 into ex[]
// (LDS, ne doubles), then k rounds of a wave-wide best-of by (ex descending, index ascending); the u64 bit pattern of a
// non-negative double orders like the double.  The chosen experts go to top[t] (LDS), unused ranks hold 0xffffffff.  Kept
// as compact loops: this is the fallback of route_ids and code size matters more than its speed.
__device__ __attribute__((noinline)) void route_ids_exact(const float* lg, u32 ne, u32 k, u32 lane, double* ex, u32* top) {
    float mx = -3.402823466e+38f;
    for (u32 i = lane; i < ne; i += 64) mx = fmaxf(mx, lg[i]);
    mx = wave_max_f32(mx);
#pragma unroll 1
    for (u32 i = lane; i < ne; i += 64) ex[i] = exp((double) (lg[i] - mx));
    u32 taken = 0;   // bit q: expert lane + 64 q is chosen
#pragma unroll 1
    for (u32 t = 0; t < k; t++) {
        u64 best = 0;   // key + 1 of the best entry still there (0: nothing left)
        u32 bi = 0xffffffffu;
#pragma unroll 1
        for (u32 q = 0; q * 64 + lane < ne; q++) {
            if ((taken >> q) & 1u) continue;
            const u64 key = __builtin_bit_cast(u64, ex[q * 64 + lane]) + 1;
            if (key > best) {
                best = key;
                bi = q * 64 + lane;
            }
        }
        const u64 wmax = wave_max_u64(best);
        const u32 win = wave_min_u32((wmax != 0 && best == wmax) ? bi : 0xffffffffu);
        if (lane == 0) top[t] = win;
        if (win != 0xffffffffu && (win & 63u) == lane) taken |= 1u << (win >> 6);
    }
    for (u32 t = k + lane; t < 16; t += 64) top[t] = 0xffffffffu;
}

// The f32 fast path of the same selection.  d = logit - max in f32 is what the reference feeds to exp (forward.rs:1101), and
// exp is strictly increasing on f32 inputs in [-700, -2^-26], so there the order by d is the order by ex; outside (a second
// logit within 2^-26 of the maximum, or a chosen expert 700 below it, where distinct d can round to one ex) the caller
// falls back to route_ids_exact.  Keys are (~bits(d)) << 32 | ~index: one u64 maximum gives the best d and the lowest
// index.  Each lane keeps its 8 keys sorted, so a round is one wave maximum and a shift in the winning lane.
// Returns false when the fallback is needed; top[] (LDS) as route_ids_exact.
__device__ __forceinline__ bool route_ids_fast(const float* lg, u32 ne, u32 k, u32 lane, u32* top) {
    // all eight loads are issued before the first one is waited for: a load behind a branch would be waited for on the
    // spot, eight memory round trips in a row; out-of-range lanes read the last logit instead and drop it
    float lv[8];
#pragma unroll
    for (int q = 0; q < 8; q++) lv[q] = lg[min(q * 64 + lane, ne - 1)];
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int q = 0; q < 8; q++)
        if (q * 64 + lane < ne) mx = fmaxf(mx, lv[q]);
    mx = wave_max_f32(mx);
    u64 c[8];
    bool risky = false;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const u32 i = q * 64 + lane;
        const float d = lv[q] - mx;
        const bool there = i < ne;
        risky = risky || (there && ((d < 0.0f && d > -1.4901161e-08f) || d != d));
        c[q] = there ? ((u64) (~f32_bits(d)) << 32) | (u64) (0xffffffffu - i) : 0ull;
    }
    if (__builtin_amdgcn_ballot_w64(risky) != 0) return false;
    // sort the lane's 8 keys, largest first (a 19-exchange network)
#define SZ_CX(a, b)                         \
    {                                       \
        const u64 hi = c[a] > c[b] ? c[a] : c[b]; \
        const u64 lo = c[a] > c[b] ? c[b] : c[a]; \
        c[a] = hi;                          \
        c[b] = lo;                          \
    }
    SZ_CX(0, 1) SZ_CX(2, 3) SZ_CX(4, 5) SZ_CX(6, 7)
    SZ_CX(0, 2) SZ_CX(1, 3) SZ_CX(4, 6) SZ_CX(5, 7)
    SZ_CX(1, 2) SZ_CX(5, 6) SZ_CX(0, 4) SZ_CX(3, 7)
    SZ_CX(1, 5) SZ_CX(2, 6)
    SZ_CX(1, 4) SZ_CX(3, 6)
    SZ_CX(2, 4) SZ_CX(3, 5)
    SZ_CX(3, 4)
#undef SZ_CX
    bool deep = false;
#pragma unroll 1
    for (u32 t = 0; t < k; t++) {
        const u64 best = wave_max_u64(c[0]);
        u32 idx = 0xffffffffu;
        if (best != 0) {
            idx = 0xffffffffu - (u32) best;
            // bits(d) of the winner above bits(-700): exp is in its subnormal tail there
            deep = deep || (~(u32) (best >> 32)) > 0xc42f0000u;
            if ((idx & 63u) == lane) {
#pragma unroll
                for (int q = 0; q < 7; q++) c[q] = c[q + 1];
                c[7] = 0;
            }
        }
        if (lane == 0) top[t] = idx;
    }
    for (u32 t = k + lane; t < 16; t += 64) top[t] = 0xffffffffu;
    return !deep;
}

// The six steps with the lane move folded into the maximum (one instruction a step instead of a copy, a move and a
// maximum; written out because the compiler does not fold a move whose unwritten lanes must keep their value).  A lane
// whose source lies outside its row, or whose row the mask leaves out, is not written and keeps its own value; a DPP read
// of a register needs two wait states after the instruction that wrote it.
__device__ __forceinline__ u32 wave_max_u32(u32 v) {
    asm volatile(
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return __builtin_amdgcn_readlane(v, 63);
}

// The same selection on 32-bit keys, less than half the instructions: the upper 23 bits of ~bits(d) above the 9 bits of
// ~index (ne <= 512).  Dropping the low 9 bits of d keeps the order of any two logits whose d differ above them; where two
// neighbours of the first k + 1 in key order agree in all 23 bits (a tie, or a difference below 2^-14 relative) the order
// by index may be wrong, so k + 1 rounds are run, every round's best is compared with the one before, and the caller falls
// back to route_ids_fast on a match.  The other two conditions are route_ids_fast's.
__device__ __forceinline__ bool route_ids_fast32(const float* lg, u32 ne, u32 k, u32 lane, u32* top) {
    float lv[8];
#pragma unroll
    for (int q = 0; q < 8; q++) lv[q] = lg[min(q * 64 + lane, ne - 1)];
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int q = 0; q < 8; q++)
        if (q * 64 + lane < ne) mx = fmaxf(mx, lv[q]);
    mx = wave_max_f32(mx);
    u32 c[8];
    bool risky = false;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const u32 i = q * 64 + lane;
        const float d = lv[q] - mx;
        const bool there = i < ne;
        risky = risky || (there && ((d < 0.0f && d > -1.4901161e-08f) || d != d));
        c[q] = there ? ((~f32_bits(d)) & 0xfffffe00u) | (0x1ffu - i) : 0u;
    }
    if (__builtin_amdgcn_ballot_w64(risky) != 0) return false;
#define SZ_CX(a, b)                         \
    {                                       \
        const u32 hi = max(c[a], c[b]);     \
        c[b] = min(c[a], c[b]);             \
        c[a] = hi;                          \
    }
    SZ_CX(0, 1) SZ_CX(2, 3) SZ_CX(4, 5) SZ_CX(6, 7)
    SZ_CX(0, 2) SZ_CX(1, 3) SZ_CX(4, 6) SZ_CX(5, 7)
    SZ_CX(1, 2) SZ_CX(5, 6) SZ_CX(0, 4) SZ_CX(3, 7)
    SZ_CX(1, 5) SZ_CX(2, 6)
    SZ_CX(1, 4) SZ_CX(3, 6)
    SZ_CX(2, 4) SZ_CX(3, 5)
    SZ_CX(3, 4)
#undef SZ_CX
    bool bad = false;
    u32 before = 0;
#pragma unroll 1
    for (u32 t = 0; t <= k; t++) {
        const u32 best = wave_max_u32(c[0]);
        bad = bad || (t > 0 && best != 0 && (best >> 9) == (before >> 9));
        if (t == k) break;
        before = best;
        // the winner's truncated bits(d) at or above bits(-700): exp is in its subnormal tail there
        bad = bad || (best != 0 && ((~best) & 0xfffffe00u) >= 0xc42f0000u);
        if (best != 0 && c[0] == best) {
#pragma unroll
            for (int q = 0; q < 7; q++) c[q] = c[q + 1];
            c[7] = 0;
        }
        if (lane == 0) top[t] = best != 0 ? 0x1ffu - (best & 0x1ffu) : 0xffffffffu;
    }
    for (u32 t = k + lane; t < 16; t += 64) top[t] = 0xffffffffu;
    return !bad;
}

// The chosen experts of one token into top[0..16) (LDS), exactly as forward::route orders them: the fast paths where they
// are safe, else the f64 one (which needs ex, ne doubles of LDS).  The wave must fence before other waves read top.
__device__ __attribute__((noinline)) void route_ids_careful(const float* lg, u32 ne, u32 k, u32 lane, double* ex, u32* top) {
    if (!route_ids_fast(lg, ne, k, lane, top)) route_ids_exact(lg, ne, k, lane, ex, top);
}
__device__ __forceinline__ void route_ids(const float* lg, u32 ne, u32 k, u32 lane, double* ex, u32* top) {
    if (!route_ids_fast32(lg, ne, k, lane, top)) route_ids_careful(lg, ne, k, lane, ex, top);
}
// As route_ids for a caller that only reads top[t]: the 32-bit path stops after rank t + 1 (the expert of rank t is settled
// once no neighbour of it in the order ties with it; ties further down cannot change it), top[t + 1 ..] are then unset.
__device__ __forceinline__ void route_id_of_rank(const float* lg, u32 ne, u32 k, u32 t, u32 lane, double* ex, u32* top) {
    if (!route_ids_fast32(lg, ne, min(k, t + 1), lane, top)) route_ids_careful(lg, ne, k, lane, ex, top);
}

// The renormalised weights of the chosen experts top[t] (forward.rs:1143-1147): lane t < k returns the f32 weight of rank
// t (0 for an unused rank); *count gets the number of chosen experts.  z is summed over the wave as a fixed tree, not in
// index order: it only scales the weights, which are rounded to f32.
__device__ __attribute__((noinline)) float route_weights(const float* lg, u32 ne, u32 k, u32 lane, const u32* top, u32* count) {
    float lv[8];   // ne <= 512; every load issued before the first is waited for
#pragma unroll
    for (int q = 0; q < 8; q++) lv[q] = lg[min(q * 64 + lane, ne - 1)];
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int q = 0; q < 8; q++)
        if (q * 64 + lane < ne) mx = fmaxf(mx, lv[q]);
    mx = wave_max_f32(mx);
    double zl = 0.0;
#pragma unroll 1
    for (u32 q = 0; q < 8; q++) {
        float v = lv[0];   // lv[q] without a dynamic register index
#pragma unroll
        for (int s = 1; s < 8; s++) v = q == (u32) s ? lv[s] : v;
        if (q * 64 + lane < ne) zl += exp((double) (v - mx));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) zl += __shfl_xor(zl, o, SZ_WAVE);
    // lane t holds ex of rank t; tz = their sum of ex / z in rank order (a chain, as the reference sums)
    const u32 e = lane < k ? top[lane] : 0xffffffffu;
    const double mine = e != 0xffffffffu ? exp((double) (lg[e] - mx)) / zl : 0.0;
    double tz = 0.0;
    u32 kk = 0;
#pragma unroll 1
    for (u32 t = 0; t < k; t++) {
        const double v = __shfl(mine, t, SZ_WAVE);
        if (__shfl(e, t, SZ_WAVE) != 0xffffffffu) {
            tz += v;
            kk++;
        }
    }
    *count = kk;
    return e != 0xffffffffu ? (float) (mine / tz) : 0.0f;
}

// The same weights without the sum over all experts: w_t = ex_t / (sum of the chosen ex), which is what the reference's
// (ex_t / z) / (sum of the chosen ex / z) is before rounding; in f64 the two differ by a few units in the last place at
// most, far below the f32 the weights are rounded to.  Ten exponentials instead of ne: for a caller with the chosen
// experts in LDS and a wave to spare but no time.  Lane t < k returns the weight of rank t; *count as route_weights.
__device__ __forceinline__ float route_weights_chosen(const float* lg, u32 ne, u32 k, u32 lane, const u32* top, u32* count) {
    float lv[8];
#pragma unroll
    for (int q = 0; q < 8; q++) lv[q] = lg[min(q * 64 + lane, ne - 1)];
    const u32 e = lane < k ? top[lane] : 0xffffffffu;
    const float le = lg[e != 0xffffffffu ? e : 0];
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int q = 0; q < 8; q++)
        if (q * 64 + lane < ne) mx = fmaxf(mx, lv[q]);
    mx = wave_max_f32(mx);
    const double mine = e != 0xffffffffu ? exp((double) (le - mx)) : 0.0;
    double tz = 0.0;
    u32 kk = 0;
#pragma unroll 1
    for (u32 t = 0; t < k; t++) {
        const double v = __shfl(mine, t, SZ_WAVE);
        if (__shfl(e, t, SZ_WAVE) != 0xffffffffu) {
            tz += v;
            kk++;
        }
    }
    *count = kk;
    return e != 0xffffffffu ? (float) (mine / tz) : 0.0f;
}
