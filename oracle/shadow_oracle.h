/* CPU oracle for the speculative-verify hot path (quantized MoE expert products, routing, lm_head argmax, greedy
 * draft acceptance).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in scalar C++, the arithmetic of the reference's CPU
 * path so that the HIP kernels can be checked against it; only tests, the smoke check and the benchmark's
 * cpu_baseline leg may load it.  Nothing under shadow_engine_amd/ links, loads or calls it.
 *
 * Every function names the reference source it follows (paths relative to the reference checkout).  How each one is
 * pinned (golden vectors, closed forms, brute force) is listed at the top of shadow_oracle.cpp.
 */
#ifndef SHADOW_ORACLE_H
#define SHADOW_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids the hot path uses (crates/shadowzero-model/src/gguf.rs:99-140,201-212). */
#define ORC_TYPE_F32 0
#define ORC_TYPE_F16 1
#define ORC_TYPE_BF16 30
#define ORC_TYPE_Q8_0 8
#define ORC_TYPE_IQ3_S 21
/* EXL3: 1000 + 10*codebook + K (K = 1..8); 1030 + K for K + 0.5 (codebook 2 only). */
#define ORC_TYPE_EXL3(cb, k) (1000 + 10 * (cb) + (k))
#define ORC_TYPE_EXL3_HALF(k) (1030 + (k))

/* ---- half.rs ---------------------------------------------------------------------------------------------------- */
float orc_f16_to_f32(uint16_t h);          /* half.rs:4  */
uint16_t orc_f32_to_f16(float f);          /* half.rs:23 */
uint16_t orc_f64_to_f16_bits(double x);    /* exl3.rs:32 */
float orc_round_f16(double x);             /* exl3.rs:28 */

/* ---- quant.rs ---------------------------------------------------------------------------------------------------- */
/* Elements and bytes of one block of a GGUF type (0 when the type has no block layout here). */
int orc_block_layout(int ggml_type, uint64_t* elems, uint64_t* bytes);
/* quant.rs:229: whole blocks of `ggml_type` into `out` (nout must equal the weights the bytes carry). 0 = ok. */
int orc_dequantize(int ggml_type, const uint8_t* data, size_t nbytes, float* out, size_t nout);

/* ---- forward.rs: matvec / Backend --------------------------------------------------------------------------------- */
typedef struct {
    int32_t ggml_type;   /* ORC_TYPE_* */
    uint64_t cols;       /* dims[0]: GGUF row length; EXL3 in_features */
    uint64_t rows;       /* dims[1]: GGUF rows; EXL3 out_features */
    const uint8_t* bytes;
    uint64_t nbytes;
} orc_tensor;

/* CpuBackend::matvec (forward.rs:239-249): y[rows] = W x.  threads <= 0 means all hardware threads. 0 = ok. */
int orc_backend_matvec(const orc_tensor* t, const float* x, float* y, int threads);

/* ---- exl3.rs ------------------------------------------------------------------------------------------------------ */
float orc_exl3_codebook(int cb, uint32_t state);                                  /* exl3.rs:66-103 */
void orc_exl3_tile_pos(int p, int* row, int* col);                                /* exl3.rs:106 */
uint32_t orc_exl3_state(const uint16_t* tile, int bits, int half, int t);         /* exl3.rs:174 */
void orc_exl3_decode_tile(const uint16_t* tile, int bits, int half, int cb, float* out256);       /* exl3.rs:190 */
void orc_exl3_decode_tile_fast(const uint16_t* tile, int bits, int half, int cb, float* out256);  /* exl3.rs:375 */
uint64_t orc_exl3_blob_len(uint64_t in_f, uint64_t out_f, int bits, int half);    /* exl3.rs:390 */
void orc_wht128(float* v128);                                                     /* exl3.rs:583 */
/* W_hat[in][out] straight from the trellis (exl3.rs:242) and W = diag(suh) H W_hat H diag(svh) (exl3.rs:259). */
int orc_exl3_reconstruct(uint64_t in_f, uint64_t out_f, int bits, int half, int cb, const uint8_t* blob, uint64_t nbytes,
                         int inner_only, float* w);
/* exl3.rs:528 */
int orc_exl3_matvec_blob(uint64_t in_f, uint64_t out_f, int bits, int half, int cb, const uint8_t* blob, uint64_t nbytes,
                         const float* x, float* y, int threads);

/* ---- forward.rs: router and MoE layer ------------------------------------------------------------------------------ */
/* route_into (forward.rs:1088-1153): the k most probable experts, most probable first (lower index at a tie), with
 * renormalised weights in f64.  Returns how many were written (min(k, ne)). */
int orc_route(const float* logits, int ne, int k, uint32_t* idx, double* w);

float orc_silu(float x);      /* forward.rs:266 (f64 exp inside) */
float orc_sigmoid(float x);   /* forward.rs:262 */

/* rmsnorm over each `group`-wide slice on its own (forward.rs:251-260): out = (x * 1/sqrt(mean(x^2) + eps)) as f32 * w, the
 * mean and the scaling in f64. */
void orc_rmsnorm_groups(const float* x, const float* w, size_t n, size_t group, float eps, float* out);
/* A hyper-connection read (forward.rs:797-817) of the residual streams r[streams * hidden]: rn = rmsnorm_groups(r, norm);
 * down = silu(W_down rn / streams); mix = sigmoid(W_up down); u[i] = sum_s mix[s h + i] rn[s h + i] / streams;
 * g[s] = 2 sigmoid(W_inject rn / streams) when inject is given.  Matrices are row-major tensors of any type the backend
 * multiplies: down [rank][streams*hidden], up [streams*hidden][rank], inject [streams][streams*hidden]. */
int orc_hc_read(const float* r, size_t hidden, size_t streams, size_t rank, float eps, const float* norm_w, const orc_tensor* down,
                const orc_tensor* up, const orc_tensor* inject, float* u, float* g, int threads);
/* hc_write (forward.rs:1078-1084): r[s h + i] += g[s] * y[i]. */
void orc_hc_write(float* r, const float* g, const float* y, size_t hidden, size_t streams);

typedef struct {
    int32_t gate_up_type;        /* type of gate and up (same type and shape) */
    int32_t down_type;
    uint64_t hidden, ff;         /* gate/up: hidden -> ff; down: ff -> hidden */
    uint64_t gate_bytes, up_bytes, down_bytes;   /* sizes of the three parts of an expert blob [gate|up|down] */
} orc_expert_shape;

/* Session::moe (forward.rs:1009-1034) for one token, with the router logits and the shared expert's gate logit given.
 * experts[e] points at expert e's contiguous [gate|up|down]; shared may be NULL (no shared expert).
 * route_idx/route_w (k entries, may be NULL) receive the routing as f32-rounded weights like the reference records. */
int orc_moe_token(const orc_expert_shape* shape, const uint8_t* const* experts, int ne, int k, const float* logits,
                  const orc_expert_shape* shared_shape, const uint8_t* shared, float shared_gate_logit,
                  const float* u, float* y, uint32_t* route_idx, float* route_w, int threads);

/* ---- cpu_expert*.rs: the int8-activation expert arithmetic (prefill chunk) ---------------------------------------- */
/* cpu_expert_avx512.rs:25-42: per block of `blk` values d = amax/127, q = clamp(round_half_away(v/d)). */
void orc_quantize_act(const float* x, size_t n, size_t blk, int8_t* q, float* d, int32_t* sums);
/* cpu_expert.rs:99-110: an IQ3_S block as 256 signed int8 (grid * sign) and 8 sub-block scales d*(1+2s). */
void orc_iq3s_int8(const uint8_t* block110, int8_t* q256, float* s8);
/* One row of an IQ3_S matrix dotted with int8 activations quantized per 32: sum over 32-blocks of
 * (s_w * d_x) * (float)(int32 dot), f32 accumulation in block order.  isums (may be NULL) gets the int32 dots. */
float orc_iq3s_row_dot_q8(const uint8_t* row, size_t cols, const int8_t* q, const float* d, int32_t* isums);
/* One expert on int8 activations: gate/up dots, SwiGLU with f32 exp (cpu_expert.rs:217), H re-quantized per 32,
 * down dots.  x_q/x_d: the token's quantized activations; out[hidden] unweighted (cpu_expert.rs:243-339). */
int orc_expert_int8(const uint8_t* expert, uint64_t hidden, uint64_t ff, const int8_t* x_q, const float* x_d, float* out,
                    float* act_out /* ff, may be NULL */);

/* ---- sampler.rs / engine.rs: argmax, top-64, greedy acceptance ----------------------------------------------------- */
uint32_t orc_argmax(const float* v, size_t n);                                   /* sampler.rs:99 (first maximum) */
/* value descending, id ascending, NaN as -inf (crates/shadowzero-cuda/tests/topk.rs:77-79). */
void orc_topk(const float* row, size_t n, int k, float* vals, uint32_t* ids);
/* engine.rs:2377-2408 without sampler or stop tokens: keep = 1 + leading drafts that equal the model's choice. */
/* The lookup drafter (crates/shadowzero-serve/src/engine.rs:828-839): drafted tokens into out[k], their number returned. */
int orc_lookup_draft(const uint32_t* hist, size_t n_hist, int k, const uint32_t* lens, int n_lens, uint32_t* out);
int orc_accept(const uint32_t* want, const uint32_t* drafts, int n_drafts);

/* ---- the inexact 2-bit lm_head screen: kernels/exl3.cu:916-987 (builder), kernels/forward.cu:4371-4622 (input codes,
 * block maxima, choice of blocks).  The reference has these as CUDA kernels only; their arithmetic is restated. ---------- */
/* w_q2: no/128 * ni/128 * 2 * 128 groups of four u32; w_sc: no * ni/128 f16 bit patterns. */
int orc_q2_proxy_build(uint64_t ni, uint64_t no, int bits, const uint8_t* blob, uint64_t nbytes, uint32_t* w_q2, uint16_t* w_sc);
/* One input row: xq[ni/4] packed int8 codes, x_sc[ni/128], x_corr[ni/128]. */
void orc_q2_proxy_quant_x(const uint8_t* blob, const float* x, uint64_t ni, uint32_t* xq, float* x_sc, float* x_corr);
/* One input row: bmax[n_ob] = the largest screen score of every 128-output block. */
void orc_q2_proxy_bmax(const uint32_t* w_q2, const uint16_t* w_sc, const uint32_t* xq, const float* x_sc, const float* x_corr,
                       uint64_t n_ob, uint64_t ni, float* bmax);
/* bmax[m][n_ob] -> sel[0] = number of chosen blocks (at most max_sel), sel[1 ..] the blocks ascending; returns the number marked. */
uint32_t orc_q2_proxy_pick(const float* bmax, uint32_t m, uint32_t n_ob, uint32_t k_blk, uint32_t max_sel, uint32_t* sel);

int orc_hardware_threads(void);

#ifdef __cplusplus
}
#endif
#endif
