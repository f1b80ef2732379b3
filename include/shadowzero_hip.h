/* shadowzero_hip: the speculative-verify hot path of ShadowZero on AMD MI355X (gfx950), as a C ABI.
 *
 * Calling convention (the reference's native-DLL style, crates/shadowzero-cuda/src/mmq.rs:9-16 and fused.rs:9-16): device
 * addresses are uint64_t of the caller's current HIP context (the device's primary context), sizes are 64-bit, a stream
 * is a hipStream_t passed as uint64_t (0 = the null stream), every call returns 0 on success and nonzero on failure with
 * the reason in sz_last_error().  Device entry points are asynchronous on the stream they are given unless they say
 * otherwise.  The library binds libamdhip64 and libhiprtc at run time (dlopen); it links neither.
 *
 * Paths in the comments are relative to the reference checkout.
 */
#ifndef SHADOWZERO_HIP_H
#define SHADOWZERO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (crates/shadowzero-model/src/gguf.rs:99-140, 201-212) of the formats the path runs on. */
#define SZ_TYPE_F32 0   /* unquantized matrices: the router, the shared expert's gate (quant.rs:237-239) */
#define SZ_TYPE_F16 1
#define SZ_TYPE_BF16 30
#define SZ_TYPE_Q8_0 8
#define SZ_TYPE_IQ3_S 21
#define SZ_TYPE_EXL3(k) (1020 + (k)) /* codebook 2 ("mul1"), K = 1..8 bits a weight */
#define SZ_TYPE_EXL3_HALF(k) (1030 + (k)) /* K + 1/2 bits a weight, K = 1..3 (Rate::end_bit, exl3.rs:164) */

/* The last error of the calling thread ("" if none).  Replaces the Result<_, String> / CudaError{code, call, name} of
 * crates/shadowzero-cuda/src/driver.rs:224-237. */
const char* sz_last_error(void);

/* ---- B0: the driver binding (driver.rs:247-689, nvrtc.rs:180-256) ------------------------------------------------- */
/* Binds libamdhip64 (SHADOWZERO_HIP_LIB overrides the name), hipInit, selects `device`, loads the kernel programs from
 * the code-object cache next to the library (SHADOWZERO_KERNEL_CACHE overrides; a miss compiles with hiprtc and fills
 * the cache).  Idempotent.  Context::new + Program::load (driver.rs:257, kernels.rs:532). */
int32_t sz_init(int32_t device);
int32_t sz_device_count(int32_t* count);                         /* driver.rs:257 (cuDeviceGetCount); needs no sz_init */
int32_t sz_device_name(char* buf, uint64_t len);                 /* cuDeviceGetName */
int32_t sz_mem_info(uint64_t* free_bytes, uint64_t* total_bytes);/* cuMemGetInfo */
int32_t sz_malloc(uint64_t* dev, uint64_t bytes);                /* Context::alloc, driver.rs:300 */
int32_t sz_free(uint64_t dev);
int32_t sz_upload(uint64_t dev, const void* host, uint64_t bytes);                 /* DeviceBuffer::upload (synchronous) */
int32_t sz_download(void* host, uint64_t dev, uint64_t bytes);                     /* DeviceBuffer::download (synchronous) */
int32_t sz_memset(uint64_t dev, int32_t byte, uint64_t bytes, uint64_t stream);   /* DeviceBuffer::zero, driver.rs:419 (cuMemsetD8); here asynchronous on the stream, a launch of the library's own (fill_bytes), so it may be captured */
int32_t sz_stream_create(uint64_t* stream);                      /* Context::stream, driver.rs:397 */
int32_t sz_stream_destroy(uint64_t stream);
int32_t sz_stream_synchronize(uint64_t stream);
int32_t sz_synchronize(void);                                    /* Context::synchronize */
int32_t sz_event_create(uint64_t* event);                        /* Context::event, driver.rs:410 */
int32_t sz_event_destroy(uint64_t event);
int32_t sz_event_record(uint64_t event, uint64_t stream);
int32_t sz_stream_wait_event(uint64_t stream, uint64_t event);  /* Stream::wait_event, driver.rs:354,586: work queued on stream after this call waits for the event's last record */
int32_t sz_event_synchronize(uint64_t event);
int32_t sz_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms);
int32_t sz_capture_begin(uint64_t stream);                       /* Stream::begin_capture, driver.rs:590 */
int32_t sz_capture_end(uint64_t stream, uint64_t* graph_exec);   /* end_capture + instantiate */
int32_t sz_graph_launch(uint64_t graph_exec, uint64_t stream);   /* Graph::launch, driver.rs:629 */
int32_t sz_graph_destroy(uint64_t graph_exec);

/* ---- B3: the kernel registry and the checked launch (kernels.rs:9-43, 546-598) ------------------------------------ */
enum { SZ_ARG_PTR = 0, SZ_ARG_U32 = 1, SZ_ARG_I32 = 2, SZ_ARG_U64 = 3, SZ_ARG_F32 = 4 };
typedef struct {
    int32_t kind;   /* SZ_ARG_* */
    int32_t pad;
    uint64_t value; /* the argument in the low bytes of an 8-byte little-endian slot, as kernels.rs:560-566 packs it */
} sz_arg;
/* Parameter kinds in the registry: a device pointer argument satisfies both pointer kinds. */
enum { SZ_P_PTR = 0, SZ_P_CONSTPTR = 1, SZ_P_U32 = 2, SZ_P_I32 = 3, SZ_P_U64 = 4, SZ_P_F32 = 5 };
/* Program::launch: refuses an unknown name, a wrong argument count or a kind mismatch before anything reaches the driver. */
int32_t sz_launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz,
                  uint32_t shared_bytes, uint64_t stream, const sz_arg* args, int32_t nargs);
int32_t sz_kernel_count(void);
/* Entry i of the registry: its name, its file, and its parameter kinds (up to max_params written). Needs no device. */
int32_t sz_kernel_info(int32_t i, const char** name, const char** file, int32_t* nparams, int32_t* kinds, int32_t max_params);
uint64_t sz_launch_count(void);                                  /* kernels.rs:519 LAUNCHES */
/* Per-kernel GPU time (SHADOWZERO_KTIME=1 of kernels.rs:527-536, 570-583): while enabled, every launch outside a stream
 * capture whose name starts with `prefix` ("" = all) sits between two events on its stream.  sz_ktime_begin resets the
 * records; sz_ktime_entry(i, ..) waits for the device and returns kernel i's launches and total milliseconds
 * (nonzero when i is past the last kernel); sz_ktime_end stops timing and frees the events. */
int32_t sz_ktime_begin(const char* prefix);
int32_t sz_ktime_entry(int32_t i, const char** name, uint64_t* launches, double* total_ms);
int32_t sz_ktime_end(void);
/* The cache key (64 hex digits + NUL into `hex65`) of kernel file `file`: SHA-256 over the assembled source, the compile
 * options, the target and the way it is built, as nvrtc.rs:185-194.  sz_program_cache_key names the object that hipcc
 * builds ahead of time with sz_program_aot_options(file) (the library's options plus the file's `// hipcc:` lines),
 * sz_program_cache_key_rtc the one the library compiles itself with hiprtc on a cache miss (the library's options only): the
 * two are different binaries and never share a name.  Need no device. */
int32_t sz_program_cache_key(const char* file, char* hex65);
int32_t sz_program_cache_key_rtc(const char* file, char* hex65);
const char* sz_program_aot_options(const char* file);
int32_t sz_program_file_count(void);
const char* sz_program_file_name(int32_t i);
/* The directory code objects are cached in, and the compile options one `hipcc --genco` needs to fill it ahead of time
 * (space-separated).  Need no device. */
const char* sz_cache_dir(void);
const char* sz_compile_options(void);
/* Writes the assembled source of `file` (prelude + headers + file, what the key hashes and the compiler sees) to `path`. */
int32_t sz_program_write_source(const char* file, const char* path);
/* Compiles `source` for the current device with hiprtc and loads nothing: the run-time compile path on its own
 * (nvrtc.rs:180).  The log (errors included) is returned in a thread-local buffer through *log. */
int32_t sz_rtc_compile(const char* name, const char* source, uint64_t* code_bytes, const char** log);

/* ---- B1: Backend::matvec (crates/shadowzero-model/src/forward.rs:231-236, crates/shadowzero-cuda/src/backend.rs:57-101) */
typedef struct sz_backend sz_backend;
sz_backend* sz_backend_new(uint64_t resident_budget_bytes);      /* GpuBackend::new, backend.rs:27 */
void sz_backend_free(sz_backend*);
/* y[rows] = W x.  GGUF types: `bytes` is rows whole rows of `cols` weights; EXL3: a blob with in = cols, out = rows.  A
 * non-null `key` names bytes that never change: uploaded once and kept resident within the budget.  Host pointers in,
 * host pointers out, synchronous, like the reference's. */
int32_t sz_matvec(sz_backend*, int32_t ggml_type, uint64_t cols, uint64_t rows, const void* bytes, uint64_t nbytes, const char* key,
                  const float* x, float* y);
uint64_t sz_backend_resident_bytes(const sz_backend*);
uint64_t sz_backend_uploads(const sz_backend*);

/* ---- B4: device entry points (device addresses in and out, asynchronous on `stream`) ------------------------------- */
/* Whole blocks (GGUF) or a whole blob (EXL3, W_hat[in][out] in the rotated basis, exl3.rs:242) to f32: the bit-exact
 * dequantization hooks (crates/shadowzero-cuda/tests/dequant.rs, tests/exl3.rs:65-77).  EXL3: cols = in, rows = out. */
int32_t sz_dequantize(int32_t ggml_type, uint64_t w, uint64_t out_f32, uint64_t cols, uint64_t rows, uint64_t stream);
int32_t sz_exl3_codebook(uint64_t out_f32_65536, uint64_t stream);
/* y_j = W x_j, j < m <= 8 (matvec_cols_*, kernels/matvec.cu:677; matvec_cols_exl3_*, kernels/exl3.cu:260): x rows xs floats
 * apart, y rows ys floats apart.  `scratch`/`scratch_bytes`: device workspace, sz_matvec_cols_scratch() bytes. */
uint64_t sz_matvec_cols_scratch(int32_t ggml_type, uint64_t cols, uint64_t rows, uint32_t m);
int32_t sz_matvec_cols(int32_t ggml_type, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys,
                       uint32_t m, uint64_t scratch, uint64_t scratch_bytes, uint64_t stream);
/* sz_matvec_cols without a workspace argument and without any allocation.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, serving loops, harnesses that forbid
 * hipMalloc).  The workspace is a device array of SZ_STATIC_WORKSPACE_BYTES inside the library, one copy on every GPU the
 * library runs on, held until the process ends; a product whose sz_matvec_cols_scratch() is larger is refused with an
 * error before anything is launched (GGUF and unquantized types need none; an EXL3 expert projection needs tens of KB).
 * Results are those of sz_matvec_cols, bit for bit.  All calls on one GPU share the array: calls that overlap in time on
 * one GPU (two streams) race on it; calls on one stream are ordered and need nothing cleared between them. */
#define SZ_STATIC_WORKSPACE_BYTES (4u << 20)
int32_t sz_matvec_cols_static(int32_t ggml_type, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys,
                              uint32_t m, uint64_t stream);

/* ---- B2: the session's verify-path operations (crates/shadowzero-cuda/src/session.rs:6076, 8222-8285, 8871, 7034-7052) */
typedef struct {
    uint32_t hidden;     /* 2048 */
    uint32_t ff;         /* expert intermediate, 512 */
    uint32_t n_expert;   /* <= 512 */
    uint32_t top_k;      /* <= 16 */
    uint32_t n_layers;
    uint32_t vocab;      /* rows of the head */
    uint32_t max_rows;   /* tokens of a verify batch, <= 8 (MAX_VERIFY, session.rs:271) */
    uint32_t reserved;
} sz_session_config;
typedef struct sz_session sz_session;
sz_session* sz_session_new(const sz_session_config*);            /* allocates the batch buffers; NULL + sz_last_error on failure */
void sz_session_free(sz_session*);
/* Layer l's resident experts: expert e is the contiguous [gate|up|down] at experts + e * stride (session.rs:9024), all of
 * one type; `shared` (0: none) is the shared expert in the same layout and of type shared_type. */
int32_t sz_session_set_layer(sz_session*, uint32_t layer, int32_t expert_type, uint64_t experts, uint64_t stride, int32_t shared_type,
                             uint64_t shared);
/* The same with `gap` bytes (a multiple of 4) between an expert's projections: [gate | gap | up | gap | down], the shared
 * expert's alike.  No counterpart in the reference, whose experts are contiguous: a layout for this memory.  An EXL3
 * projection's trellis begins 2 (in + out) + 4 bytes into its blob (exl3.rs:390-393), so in the contiguous layout every row
 * segment a launch fetches lies 4, 8 or 12 bytes off the 128-byte lines of memory and touches one line more than it fills
 * (12 to 25 % more bytes fetched).  sz_layer_spacing gives the `lead` (bytes past a 128-byte boundary at which the first
 * expert, and the shared one, should start) and the `gap` that put every trellis of a layer on a line, given a stride that
 * is a multiple of 128; both are 0 for GGUF types.  sz_exl3_layer_layout and sz_exl3_stage_layer use them. */
int32_t sz_session_set_layer_spaced(sz_session*, uint32_t layer, int32_t expert_type, uint64_t experts, uint64_t stride, uint64_t gap,
                                    int32_t shared_type, uint64_t shared);
void sz_layer_spacing(int32_t expert_type, uint64_t hidden, uint64_t ff, uint32_t* lead, uint32_t* gap);
/* output.weight, vocab x hidden: Q8_0, IQ3_S, F32, F16 or BF16 rows, or an EXL3 blob at a whole bit rate (in = hidden, out =
 * vocab, both multiples of 128; the head of an EXL3 checkpoint, session.rs:7179-7187).  The arg-max (sz_head_argmax,
 * sz_verify_round) is fused into the product for Q8_0 and EXL3; the other types go through their logits, kept in a buffer
 * this call allocates (max_rows x vocab floats), as the reference's mv_cols + topk_rows_at do (session.rs:7034-7052). */
int32_t sz_session_set_head(sz_session*, int32_t ggml_type, uint64_t w);
/* LDS a workgroup of the EXL3 head's kernel takes for m rows (0 for another type): the head entry points refuse a call
 * whose need is above a compute unit's 160 KiB (hidden 4096 takes all 8 rows at any rate, hidden 8192 up to 4), and
 * sz_session_set_head a head that cannot take one row.  No counterpart in the reference (its kernels take 64 rows in registers). */
uint32_t sz_exl3_head_lds_bytes(int32_t type, uint32_t hidden, uint32_t m);
/* The optional, INEXACT 2-bit screen of an EXL3 head for the top-64 hand-off (HeadProxy, session.rs:428-441, built at
 * session.rs:2631-2674 by exl3_build_q2_proxy_K, kernels/exl3.cu:916-996; used by head_top_at, session.rs:5952-6022): off by
 * default and after every sz_session_set_head, as the reference's exact mode has it (session.rs:786).  k_blk > 0 builds the
 * 2-bit copy of the current head (vocab * hidden / 4 bytes + an f16 scale per output and 128 inputs; hidden <= 4096) and
 * makes sz_head_top score every output with it, compute only the k_blk best 128-output blocks of every row exactly (k_blk
 * is clamped to [16, vocab / 128] as SHADOWZERO_HEAD_KBLK is, 128 there by default) and take the top 64 among those: the
 * values are the exact head's bit for bit, but an output outside the chosen blocks cannot appear.  sz_head_argmax,
 * sz_head_logits and sz_verify_round never use it.  k_blk = 0 turns it off again. */
int32_t sz_session_set_head_proxy(sz_session*, uint32_t k_blk);
/* How a layer of EXL3 experts at a whole bit rate multiplies in sz_moe_layer_verify, sz_moe_block_verify and sz_verify_round
 * (the reference's choice between its exact kernels and mma_grouped_exl3_K, kernels/exl3.cu:682-725, which `--exact` and
 * `tensor_prompt` make, session.rs:1741, 1817): 0, the default, the exact kernels (every weight the codebook's f16, f32
 * multiply-adds in input order, a work item a (token, expert) pair); 1 the matrix cores on the codebook's own f16 values, a
 * work item a distinct expert with its tokens on the rows of the matrix instruction (only the order of the f32 additions and
 * the 22 bits kept of an input differ); 2 the matrix cores on the linearised codebook (a weight's rounding to f16 is skipped:
 * outputs within 1e-3 relative L2 of the exact ones, about 4e-4 measured); 3 the exact kernels' launches and decode with
 * the rotated inputs rounded to f16, two products an instruction (about 4e-4 as well).  Routing ids, their order and the
 * weights are the same bits in every mode.  Half-integer rates always take the exact kernels.  On an MI355X modes 1 and 2 are
 * slower than the exact kernels for batches of up to 8 rows and mode 3 is 1.5 % faster.  Environment SHADOWZERO_EXPERT_MODE
 * sets a new session's mode. */
int32_t sz_session_set_expert_mode(sz_session*, int32_t mode);
/* 0: sz_verify_round launches its kernels one by one instead of replaying a captured graph (default 1). */
int32_t sz_session_set_graph(sz_session*, int32_t enabled);
/* moe_batch_resident (session.rs:8222): y[m][hidden] = the MoE block of layer l on u[m][hidden], from the router logits
 * rl[m][n_expert] and the shared expert's gate logits sgl[m] (moe_router_batch's outputs, session.rs:7868). */
int32_t sz_moe_layer_verify(sz_session*, uint32_t layer, uint32_t m, uint64_t u, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t stream);
/* Layer l's router ffn_gate_inp.weight [n_expert][hidden] and shared-expert gate ffn_gate_inp_shexp.weight [1][hidden]
 * (forward.rs:1013, 1033), unquantized (F32, F16 or BF16), resident; gate_w = 0: the layer has no shared expert gate. */
int32_t sz_session_set_router(sz_session*, uint32_t layer, int32_t router_type, uint64_t router_w, int32_t gate_type, uint64_t gate_w);
/* moe_router_batch (session.rs:7868: the router and the shared expert's gate logit for the batch's m tokens, one launch):
 * rl[m][n_expert] and sgl[m] into the session's buffers, whose device addresses sz_session_router_outputs returns. */
int32_t sz_moe_router_verify(sz_session*, uint32_t layer, uint32_t m, uint64_t u, uint64_t stream);
int32_t sz_session_router_outputs(sz_session*, uint64_t* rl, uint64_t* sgl);
/* Session::moe (forward.rs:1009-1034) for a verify batch: the router product, then sz_moe_layer_verify on its outputs. */
int32_t sz_moe_block_verify(sz_session*, uint32_t layer, uint32_t m, uint64_t u, uint64_t y, uint64_t stream);
/* The routing the last sz_moe_layer_verify of this layer-independent plan buffer made: idx[m][k], w[m][k] to the host
 * (synchronizes `stream`). */
int32_t sz_session_last_route(sz_session*, uint32_t m, uint32_t* idx, float* w, uint64_t stream);
/* The head on u[m][hidden] with the arg-max fused in (logits never written): ids[m] on the device. */
int32_t sz_head_argmax(sz_session*, uint32_t m, uint64_t u, uint64_t ids, uint64_t stream);
/* The head, then the exact top 64 of every row (value descending, id ascending; step_batch_verify_top, session.rs:6061):
 * writes top[m][128] words (64 value bits, then 64 ids) to the HOST and synchronizes, as session.rs:6034-6039 does. */
int32_t sz_head_top(sz_session*, uint32_t m, uint64_t u, uint32_t* top_host, uint64_t stream);
/* The head's logits[m][vocab] to device memory (step_batch_verify's return, session.rs:6076). */
int32_t sz_head_logits(sz_session*, uint32_t m, uint64_t u, uint64_t logits, uint64_t stream);
/* Greedy acceptance (crates/shadowzero-serve/src/engine.rs:2377-2408): ids[i] = the model's token after batch row i (host
 * arrays); *keep = 1 + leading drafts equal to ids. */
int32_t sz_verify_accept(const uint32_t* ids, const uint32_t* drafts, uint32_t n_drafts, uint32_t* keep);
/* The lookup drafter (crates/shadowzero-serve/src/engine.rs:823-839 lookup_from): for each match length of lens[] in turn, the
 * last earlier place where the history's last lens[i] tokens occur; the up to k tokens that followed it there are the
 * draft (drafts[k], *n_drafts of them; 0 when nothing matches).  Host arrays. */
int32_t sz_lookup_draft(const uint32_t* hist, uint64_t n_hist, uint32_t k, const uint32_t* lens, uint32_t n_lens, uint32_t* drafts,
                        uint32_t* n_drafts);

/* ---- the rollback point of a speculative pass: device state saved and put back, one launch each way.
 * The reference keeps the recurrent layers' states of a session in a device-side snapshot that it takes again before
 * every pass (GpuSession::snapshot_again, crates/shadowzero-cuda/src/session.rs:3407-3452) and restores when drafts are
 * rejected (restore_local's device-only branch, :3472-3510); both move all ranges with one copy_many launch over a table
 * that stays on the device while the ranges are the same (copy_many_with, :3385-3404; kernels/forward.cu:3629).
 * sz_snapshot_new: n device ranges (addrs[i], bytes[i]; empty ranges allowed) and buffers of the snapshot's own for them;
 * the ranges must not overlap each other.  take: state -> snapshot; restore: snapshot -> state (an error before the first
 * take).  Both are asynchronous on `stream` and allocate nothing.  download: the saved copy of range i to the host. */
typedef struct sz_snapshot sz_snapshot;
int32_t sz_snapshot_new(const uint64_t* addrs, const uint64_t* bytes, uint32_t n, sz_snapshot** out);
void sz_snapshot_free(sz_snapshot*);
uint64_t sz_snapshot_bytes(const sz_snapshot*);
int32_t sz_snapshot_take(sz_snapshot*, uint64_t stream);
int32_t sz_snapshot_restore(sz_snapshot*, uint64_t stream);
int32_t sz_snapshot_download(const sz_snapshot*, uint32_t i, void* host, uint64_t cap);
/* The same launch for a one-off set: ranges[3 i ..] = (dst, src, bytes) device ranges, no destination overlapping another
 * range; uploads its table, runs and waits (the entries of copy_many_with, session.rs:3387).  It allocates and
 * synchronizes the stream: it must not be called on a stream that is being captured (a snapshot object's take and
 * restore are the forms that can be). */
int32_t sz_copy_ranges(const uint64_t* ranges, uint32_t n, uint64_t stream);

/* The session's batch buffers, for tests and measurements (device addresses; the contents are those of the last call):
 * 0 the plan (chosen experts u32[m][k], weights f32[m][k], counts u32[m] for the fused layers), 1 the split-k partial sums of
 * gate and up, 2 the down products (EXL3 layers); 3 the gate and up rows, 4 the down rows of a GGUF layer's pairs; of the
 * head's 2-bit screen: 5 the levels, 6 their f16 scales, 7 the rows' int8 codes, 8 their scales, 9 their correction terms, 10 the
 * block maxima f32[m][vocab / 128], 11 the list of chosen blocks (count, then the blocks ascending), 12 the packed logits of the
 * listed blocks (rows 128 * min(m * k_use, vocab / 128) apart); of the prefill chunk of EXL3 experts: 13 the partial sums of
 * gate and up, 14 the pairs' down rows, 15 the operand rows of the down launch, 16 their factors, 17 the work items.  0 for any
 * other `which`. */
uint64_t sz_session_buffer(sz_session*, int32_t which);

/* A whole verify round over device-resident inputs: for every layer l the MoE block on u[l][m][hidden] with rl[l][m][ne]
 * and sgl[l][m] into y[l][m][hidden], then the head on head_u[m][hidden], arg-max and acceptance against drafts[m-1]
 * (device).  out[0] = keep, out[1] = bonus token, out[2..2+m) = ids (device, u32).  Captured into a HIP graph on first
 * use for these addresses and replayed afterwards. */
int32_t sz_verify_round(sz_session*, uint32_t m, uint64_t u, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t head_u, uint64_t drafts,
                        uint64_t out, uint64_t stream);

/* ---- the hyper-connection around a sublayer (forward.rs:797-817 hc_read, 1078-1084 hc_write; session.rs:7432 hc_read_batch) */
typedef struct {
    uint32_t hidden, streams, rank, max_rows;   /* max_rows <= 8 */
    float eps;
    int32_t down_type, up_type, inject_type;    /* SZ_TYPE_F32 / F16 / BF16 */
    uint64_t norm_w;     /* f32[streams * hidden] */
    uint64_t down_w;     /* [rank][streams * hidden] */
    uint64_t up_w;       /* [streams * hidden][rank] */
    uint64_t inject_w;   /* [streams][streams * hidden]; 0: this read produces no gains (the final read, forward.rs:791) */
} sz_hc_config;
typedef struct sz_hc sz_hc;
sz_hc* sz_hc_new(const sz_hc_config*);           /* resident weights by address; allocates the read's buffers */
void sz_hc_free(sz_hc*);
/* u[m][hidden] = the sublayer's input from the residual streams r[m][streams * hidden]; the per-stream gains of the write
 * that follows land in the handle's g[max_rows][streams] (sz_hc_gains).  Four launches: norm, down + inject, up, mix. */
int32_t sz_hc_read(sz_hc*, uint32_t m, uint64_t r, uint64_t u, uint64_t stream);
uint64_t sz_hc_gains(sz_hc*);
/* r[j][s * hidden + i] += g[j][s] * y[j][i]. */
int32_t sz_hc_write(uint64_t r, uint64_t g, uint64_t y, uint32_t m, uint32_t hidden, uint32_t streams, uint64_t stream);

/* ---- the prefill chunk on int8 activations (native/fused/shadowzero_fused.cu:5-9 sf_quantize/sf_group/sf_experts) --- */
/* Per-32 int8 activations: q[n], d[n/32] with d = amax/127, q = round-half-away(v/d) (cpu_expert_avx512.rs:25-42). */
int32_t sz_quantize_act(uint64_t x_f32, uint64_t n, uint64_t q_i8, uint64_t d_f32, uint64_t stream);
/* One prefill chunk through layer l (IQ3_S experts): tokens x[t][hidden] f32, routing from rl[t][n_expert], tokens grouped by
 * expert, int8 MFMA products, SwiGLU, int8 H, down, weighted combine in rank order (+ the shared expert gated by sgl[t])
 * into y[t][hidden]. */
int32_t sz_moe_prefill_chunk(sz_session*, uint32_t layer, uint32_t tokens, uint64_t x, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t stream);
/* The last chunk's intermediate device buffers, for parity tests: 0 xq int8[t][hidden], 1 xd f32[t][hidden/32], 2 tidx u32[t][k],
 * 3 w f32[t][k], 4 hq int8[pair][ff], 5 hd f32[pair][ff/32], 6 eo f32[pair][hidden] (pair = token * k + rank, then the shared
 * expert's t rows).  0 when nothing has run. */
uint64_t sz_prefill_buffer(sz_session*, int32_t which);

/* ---- B5: the checkpoint formats either side of the path (host code; no GPU is needed up to the two staging calls) ---- */
/* A ggml type id's name ("IQ3_S", "EXL3_3", "EXL3_2h", "type77") and block (elements, bytes; 0, 0 when it has none):
 * GgmlType::name / block, crates/shadowzero-model/src/gguf.rs:170-178. */
int32_t sz_type_info(uint32_t type, char* name, uint64_t len, uint64_t* block_elements, uint64_t* block_bytes);

/* The GGUF header reader (gguf.rs): key-values and the tensor table of every shard, offsets absolute; never reads tensor
 * data by itself. */
typedef struct sz_gguf sz_gguf;
typedef struct {
    uint32_t type;            /* ggml type id */
    uint32_t n_dims;
    uint32_t shard;           /* index of the file */
    uint32_t has_layout;      /* nbytes_layout is known (the type's block layout fits the row length) */
    uint64_t dims[8];         /* ggml order: dims[0] is the row length */
    uint64_t offset;          /* absolute in the shard's file */
    uint64_t nbytes_layout;
    uint64_t nbytes_span;     /* to the next tensor of the shard, or to the end of the file */
    uint64_t nbytes;          /* TensorInfo::nbytes, gguf.rs:243: the layout's when known, else the span */
} sz_tensor_info;
/* shard_paths (gguf.rs:442): the i-th file name of a model opened by `path`; *count = how many (buf may be NULL). */
int32_t sz_gguf_shard_paths(const char* path, uint32_t i, char* buf, uint64_t len, uint32_t* count);
int32_t sz_gguf_open(const char* path, sz_gguf** out);                       /* Gguf::open, gguf.rs:468: from any shard */
void sz_gguf_close(sz_gguf*);
uint64_t sz_gguf_tensor_count(const sz_gguf*);
int32_t sz_gguf_tensor_at(const sz_gguf*, uint64_t i, char* name, uint64_t name_len, sz_tensor_info* info);
int32_t sz_gguf_tensor(const sz_gguf*, const char* name, sz_tensor_info* info);   /* Gguf::tensor, gguf.rs:509; nonzero: no such tensor */
uint64_t sz_gguf_tensor_bytes(const sz_gguf*);                               /* gguf.rs:518 */
uint32_t sz_gguf_shard_count(const sz_gguf*);
int32_t sz_gguf_shard(const sz_gguf*, uint32_t i, char* path, uint64_t path_len, uint32_t* version, uint64_t* file_len, uint64_t* data_start,
                      uint64_t* alignment);
uint64_t sz_gguf_kv_count(const sz_gguf*);
int32_t sz_gguf_kv_key(const sz_gguf*, uint64_t i, char* buf, uint64_t len);   /* keys in byte order (BTreeMap) */
/* The file's value type id (0..12; 8 string, 9 array), an array's element type, and the count (array items, string bytes, else 1). */
int32_t sz_gguf_kv_type(const sz_gguf*, const char* key, uint32_t* type, uint32_t* elem_type, uint64_t* count);
int32_t sz_gguf_kv_u64(const sz_gguf*, const char* key, uint64_t* out);     /* Value::as_u64, gguf.rs:41: any integer type, not negative */
int32_t sz_gguf_arch_u64(const sz_gguf*, const char* key, uint64_t* out);   /* Gguf::arch_key, gguf.rs:504: "<architecture>.<key>" */
int32_t sz_gguf_kv_f64(const sz_gguf*, const char* key, double* out);       /* Value::as_f64, gguf.rs:55 */
int32_t sz_gguf_kv_str(const sz_gguf*, const char* key, char* buf, uint64_t len);
int32_t sz_gguf_kv_array_u64(const sz_gguf*, const char* key, uint64_t i, uint64_t* out);   /* integers and flags */
int32_t sz_gguf_kv_array_f64(const sz_gguf*, const char* key, uint64_t i, double* out);
int32_t sz_gguf_kv_array_str(const sz_gguf*, const char* key, uint64_t i, char* buf, uint64_t len);
int64_t sz_gguf_block_index(const char* name);                               /* block_index, gguf.rs:534: N of "blk.N.", or -1 */
int32_t sz_gguf_read_tensor(const sz_gguf*, const char* name, void* host, uint64_t cap);    /* Gguf::read_tensor, gguf.rs:523 */
/* Where expert e's slice of a fused [in, out, n_expert] tensor lies (Model::expert_file_range, forward.rs:477-486). */
int32_t sz_gguf_expert_range(const sz_gguf*, const char* name, uint64_t e, uint32_t* shard, uint64_t* offset, uint64_t* len);

/* The safetensors header reader (crates/shadowzero-model/src/safetensors.rs): every tensor of one or more files by name. */
typedef struct sz_safetensors sz_safetensors;
typedef struct {
    char dtype[8];            /* "F16", "I16", "BF16", ... */
    uint32_t n_dims;
    uint32_t file;            /* index into the files, sz_st_file */
    uint64_t shape[8];
    uint64_t start, end;      /* absolute byte range in that file */
} sz_st_info;
int32_t sz_st_open(const char* const* paths, uint32_t n, sz_safetensors** out);   /* SafeTensors::open, safetensors.rs:47 */
int32_t sz_st_open_dir(const char* dir, sz_safetensors** out);                    /* open_dir, safetensors.rs:56: *.safetensors in name order */
void sz_st_close(sz_safetensors*);
uint64_t sz_st_tensor_count(const sz_safetensors*);
uint32_t sz_st_file_count(const sz_safetensors*);
int32_t sz_st_file(const sz_safetensors*, uint32_t i, char* buf, uint64_t len);
int32_t sz_st_tensor_at(const sz_safetensors*, uint64_t i, char* name, uint64_t name_len, sz_st_info* info);   /* in name order */
int32_t sz_st_tensor(const sz_safetensors*, const char* name, sz_st_info* info);  /* SafeTensors::get, safetensors.rs:94 */
int32_t sz_st_read(const sz_safetensors*, const char* name, uint64_t off, uint64_t len, void* host);   /* read_range, safetensors.rs:127 */
/* An EXL3 projection `{prefix}.{trellis,suh,svh,mul1|mcg}`: its shape and ggml type id (linear_shape, exl3_model.rs:98-109;
 * bits_from_last_dim, exl3.rs:114), whether its four tensors are one range of a file in blob order (contiguous,
 * exl3_model.rs:88-95; nonzero when not), the blob's length (blob_len, exl3.rs:388) and the blob itself, [suh f16 | svh f16 |
 * 4-byte marker | trellis]: the file's range when contiguous, else put together with marker 1 (to_blob, exl3.rs:501). */
int32_t sz_exl3_shape(const sz_safetensors*, const char* prefix, uint64_t* in_features, uint64_t* out_features, int32_t* type);
int32_t sz_exl3_contiguous(const sz_safetensors*, const char* prefix, uint32_t* file, uint64_t* offset, uint64_t* len);
uint64_t sz_exl3_blob_len(uint64_t in_features, uint64_t out_features, int32_t type);
int32_t sz_exl3_read_blob(const sz_safetensors*, const char* prefix, void* host, uint64_t cap);

/* One MoE layer in the device layout sz_session_set_layer_spaced and sz_session_set_router take: expert e's
 * [gate | gap | up | gap | down] at experts_offset + e * stride, the shared expert's three alike at shared_offset, the router
 * at router_offset, the shared expert's gate at gate_offset (a type of -1: the checkpoint has none).  gap and experts_offset
 * are sz_layer_spacing's: 0 for a GGUF, what puts every trellis on a 128-byte line for an EXL3 checkpoint.  The tensors are `blk.N.ffn_{gate,up,down}_exps.weight`,
 * `ffn_*_shexp`, `ffn_gate_inp[_shexp]` of a GGUF, and `model.language_model.layers.N.mlp.{experts.E,shared_expert}.*_proj`,
 * `mlp.gate.weight`, `mlp.shared_expert_gate.weight` of an EXL3 checkpoint (exl3_map.rs:128-135). */
typedef struct {
    int32_t type, shared_type, router_type, gate_type;
    uint32_t n_expert, gap;               /* gap: bytes between an expert's projections */
    uint64_t hidden, ff;
    uint64_t gate_up_bytes, down_bytes;   /* one expert's gate (= up) and down projection */
    uint64_t shared_gate_up_bytes;
    uint64_t stride, shared_offset, router_offset, gate_offset;
    uint64_t bytes;                       /* the whole layer's buffer */
    uint64_t experts_offset;              /* where expert 0 starts */
} sz_layer_layout;
int32_t sz_gguf_layer_layout(const sz_gguf*, uint32_t layer, sz_layer_layout* out);
/* n_expert = 0: as many experts as the checkpoint has for the layer. */
int32_t sz_exl3_layer_layout(const sz_safetensors*, uint32_t layer, uint32_t n_expert, sz_layer_layout* out);
/* Reads the layer into device memory at dev (256-byte aligned, cap >= layout.bytes) through two pinned buffers, file reads on
 * several threads overlapping the copies on `stream`; returns when the bytes are on the device.  The expert slices are the
 * ranges of Model::expert_file_range (forward.rs:477-486), as experts_into_many (forward.rs:503-510) reads them. */
int32_t sz_gguf_stage_layer(const sz_gguf*, uint32_t layer, uint64_t dev, uint64_t cap, uint64_t stream);
int32_t sz_exl3_stage_layer(const sz_safetensors*, uint32_t layer, uint32_t n_expert, uint64_t dev, uint64_t cap, uint64_t stream);
/* One tensor the same way (the head's output.weight, norm weights): its file bytes to dev; and one EXL3 projection as its blob
 * (the file's range when its tensors are one, else put together, up to 64 MiB: lm_head of an EXL3 checkpoint). */
int32_t sz_gguf_stage_tensor(const sz_gguf*, const char* name, uint64_t dev, uint64_t cap, uint64_t stream);
int32_t sz_st_stage_tensor(const sz_safetensors*, const char* name, uint64_t dev, uint64_t cap, uint64_t stream);
int32_t sz_exl3_stage_blob(const sz_safetensors*, const char* prefix, uint64_t dev, uint64_t cap, uint64_t stream);

#ifdef __cplusplus
}
#endif
#endif
