// Shared device helpers for every kernel file (gfx950, wave64).  Prepended to each file before compilation.
//
// Compiled with -ffp-contract=off: a multiply followed by an add is never fused behind the code's back, so the dequant
// kernels reproduce the CPU reference's two-rounding arithmetic bit for bit; where a fused multiply-add is wanted (the
// dot products) the code says __builtin_fmaf.
#if !defined(__HIPCC_RTC__)
#include <hip/hip_runtime.h>
#endif

typedef unsigned char u8;
typedef signed char i8;
typedef unsigned short u16;
typedef unsigned int u32;
typedef int i32;
typedef unsigned long long u64;

#define SZ_WAVE 64

// a 4-dword vector that only promises 4-byte alignment (expert parts start at 4-byte offsets inside a blob)
typedef u32 u32x4a __attribute__((ext_vector_type(4), aligned(4)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float f16_to_f32(u16 h) { return (float) __builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ u32 f32_bits(float f) { return __builtin_bit_cast(u32, f); }
__device__ __forceinline__ float bits_f32(u32 b) { return __builtin_bit_cast(float, b); }

// silu and sigmoid in f32, as the reference's GPU glue (kernels/forward.cu:9-10): x / (1 + exp(-x)).
__device__ __forceinline__ float siluf_ref(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoidf_ref(float x) { return 1.0f / (1.0f + expf(-x)); }

// The value of lane (lane ^ h) for h = 1, 2, 4, 8 (row-local DPP moves) and 16, 32 (row and half swaps).
template <int h>
__device__ __forceinline__ float lane_xor(float v, u32 lane) {
    const u32 b = f32_bits(v);
    if constexpr (h == 1) return bits_f32(__builtin_amdgcn_update_dpp(b, b, 0xb1, 0xf, 0xf, false));          // quad_perm [1,0,3,2]
    else if constexpr (h == 2) return bits_f32(__builtin_amdgcn_update_dpp(b, b, 0x4e, 0xf, 0xf, false));     // quad_perm [2,3,0,1]
    else if constexpr (h == 4) {
        u32 a = __builtin_amdgcn_update_dpp(b, b, 0x124, 0xf, 0xa, false);   // row_ror:4 into lanes with bit 2 set: from lane - 4
        a = __builtin_amdgcn_update_dpp(a, b, 0x12c, 0xf, 0x5, false);       // row_ror:12 into the others: from lane + 4
        return bits_f32(a);
    } else if constexpr (h == 8) return bits_f32(__builtin_amdgcn_update_dpp(b, b, 0x128, 0xf, 0xf, false));  // row_ror:8
    else if constexpr (h == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
        return bits_f32((lane & 16) ? r[0] : r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
        return bits_f32((lane & 32) ? r[0] : r[1]);
    }
}

// Sum over the lanes of a segment of `width` lanes (a power of two, at most 64, aligned); every lane gets the sum.  A
// butterfly over lane_xor: no LDS round trips.
template <int width>
__device__ __forceinline__ float seg_sum(float v, u32 lane) {
    if constexpr (width > 1) v += lane_xor<1>(v, lane);
    if constexpr (width > 2) v += lane_xor<2>(v, lane);
    if constexpr (width > 4) v += lane_xor<4>(v, lane);
    if constexpr (width > 8) v += lane_xor<8>(v, lane);
    if constexpr (width > 16) v += lane_xor<16>(v, lane);
    if constexpr (width > 32) v += lane_xor<32>(v, lane);
    return v;
}

// The same for a width only known at run time (uniform over the wave).
__device__ __forceinline__ float seg_sum_rt(float v, u32 width, u32 lane) {
    if (width > 1) v += lane_xor<1>(v, lane);
    if (width > 2) v += lane_xor<2>(v, lane);
    if (width > 4) v += lane_xor<4>(v, lane);
    if (width > 8) v += lane_xor<8>(v, lane);
    if (width > 16) v += lane_xor<16>(v, lane);
    if (width > 32) v += lane_xor<32>(v, lane);
    return v;
}

// (value, index) maximum with ties to the lower index; a NaN counts as -inf.
__device__ __forceinline__ void argmax_merge(float& bv, u32& bi, float v, u32 i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

// The power of two that takes a largest magnitude (the bits of a non-negative float) to [2^14, 2^15), and its inverse:
// values scaled by it split into an f16 high part that cannot overflow and an f16 low part that keeps its bits down to
// 2^-39 of the largest; a largest magnitude of zero, infinity or NaN gives 1.
__device__ __forceinline__ void pow2_scale_of(u32 mx_bits, float& scale, float& inv) {
    const u32 eb = (mx_bits >> 23) & 0xffu;
    const u32 sb = (eb == 0u || eb == 255u) ? 127u : min(268u - eb, 253u);
    scale = bits_f32(sb << 23);
    inv = bits_f32((254u - sb) << 23);
}

// ---- global-to-LDS loads ------------------------------------------------------------------------------------------------
// Written as inline assembly on purpose: the compiler then keeps no count of them, so it does not hold back the first LDS
// read that follows until every one of them has landed; wait_vm is the only thing that orders them.  Consequences for the
// caller: an ordinary global load whose value is still needed must have been consumed before such a burst is issued (a
// load the compiler waits for later would wait for the whole burst, which is correct but slow), and a wave must have
// waited for its last load before it ends or lets another wave read the data.
__device__ __forceinline__ u32 lds_offset(const void* p) { return (u32) (u64) (const __attribute__((address_space(3))) void*) p; }

// One load instruction: every lane moves B bytes from its own global address to LDS address `lds` + 16 * lane (B = 16 and
// 12) or `lds` + 4 * lane (B = 4); `lds` must be wave-uniform.  A 4-byte-aligned source is enough.
template <int B>
__device__ __forceinline__ void lds_load(const void* g, u32 lds) {
    static_assert(B == 16 || B == 12 || B == 4, "sizes the chip has");
    // m0 carries the LDS address; it is put back afterwards, so the statement leaves no register changed
    u32 keep;
    lds = __builtin_amdgcn_readfirstlane(lds);   // uniform by contract; this tells the compiler so
#define SZ_LDS_LOAD(op) asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t" op " %1, off\n\ts_mov_b32 m0, %0" : "=&s"(keep) : "v"(g), "s"(lds) : "memory")
    if constexpr (B == 16) SZ_LDS_LOAD("global_load_lds_dwordx4");
    if constexpr (B == 12) SZ_LDS_LOAD("global_load_lds_dwordx3");
    if constexpr (B == 4) SZ_LDS_LOAD("global_load_lds_dword");
#undef SZ_LDS_LOAD
}

// A 4-byte global load the compiler keeps no count of (as lds_load's): the caller orders it with wait_vm and must pass the
// value through load_landed() after the wait and before its first use, which keeps the compiler from moving a use ahead.
__device__ __forceinline__ float load_f32_uncounted(const float* p) {
    float v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ u32 load_u16_uncounted(const u16* p) {
    u32 v;
    asm volatile("global_load_ushort %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void load_landed(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void load_landed(u32& v) { asm volatile("" : "+v"(v)); }

// s_waitcnt vmcnt(min(n, 63)), nothing else waited for (the counter has 6 bits; waiting for fewer is only earlier).
template <int n_>
__device__ __forceinline__ void wait_vm() {
    static_assert(n_ >= 0, "a count");
    constexpr int n = n_ < 63 ? n_ : 63;
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
    asm volatile("" ::: "memory");
}

