// The host side of the verify path above the kernels: Backend::matvec, the device entry points, and the session's MoE /
// head / acceptance operations.  Mirrors the hot subset of crates/shadowzero-cuda/src/{backend.rs,session.rs}.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "sz_internal.hpp"

namespace sz {

// ---- formats ------------------------------------------------------------------------------------------------------
bool format_of(int ty, Format& f, std::string& tag) {
    f = Format{};
    if (ty == SZ_TYPE_Q8_0) {
        f.qk = 32; f.bb = 34; tag = "q8_0";
    } else if (ty == SZ_TYPE_IQ3_S) {
        f.qk = 256; f.bb = 110; tag = "iq3_s";
    } else if (ty == SZ_TYPE_F32 || ty == SZ_TYPE_F16 || ty == SZ_TYPE_BF16) {
        f.dense = true; f.qk = 1; f.bb = ty == SZ_TYPE_F32 ? 4 : 2; tag = ty == SZ_TYPE_F32 ? "f32" : ty == SZ_TYPE_F16 ? "f16" : "bf16";
    } else if (ty >= 1021 && ty <= 1028) {
        f.exl3 = true; f.bits = ty - 1020; tag = "exl3_" + std::to_string(f.bits);
    } else if (ty >= 1031 && ty <= 1033) {
        f.exl3 = true; f.half = true; f.bits = ty - 1030; tag = "exl3h_" + std::to_string(f.bits);
    } else {
        return false;
    }
    f.tag = tag.c_str();
    return true;
}

uint64_t matrix_bytes(const Format& f, uint64_t cols, uint64_t rows) {
    if (f.exl3) return 2 * cols + 2 * rows + 4 + cols * rows * (uint64_t) (2 * f.bits + (f.half ? 1 : 0)) / 16;   // exl3.rs:390-393
    return rows * (cols / f.qk) * f.bb;
}

// Rows a workgroup of the staged GGUF kernels takes: about `lds` bytes of LDS (up to 40 KB for rows of more than 64 units), a
// multiple of 4 * (rows side by side in a wave), at most `cap` where that is such a multiple.
uint32_t rows_per_block(const Format& f, uint32_t cols, uint32_t cap, uint32_t lds) {
    if (f.exl3 || f.dense || cols == 0 || cols % f.qk || cols % 32) return 0;
    const uint32_t units = cols / 32;
    const uint32_t rb = cols / f.qk * f.bb;
    uint32_t ul = 64;                       // lanes a row takes in a wave (rows_body in kernels/matvec.hip)
    if (units < 64)
        for (ul = 1; ul < units;) ul *= 2;
    const uint32_t rg = 64 / ul;
    const uint32_t quantum = 4 * rg;
    uint32_t rpb = (lds / rb) / quantum * quantum;
    if (units > 64) rpb = 8 * rb <= 40960 ? 8 : 4;   // wide rows: 8 where they fit, so that the inputs are staged half as often (measured)
    if (rpb == 0) rpb = quantum;
    if ((uint64_t) rpb * rb + 32 + rpb * 16 > 60000) return 0;
    rpb = std::min<uint32_t>(rpb, units > 64 ? 16 : 64);   // rows_wide keeps the sums of at most 4 rows a wave
    if (rpb > cap) rpb = std::max(quantum, cap / quantum * quantum);
    return rpb;
}

// Workgroups and dynamic LDS of the unquantized-matrix kernels (dense_group in kernels/matvec.hip): a workgroup a row when
// the rows are longer than 2048, else one for every 4 to 32 rows with the inputs staged in LDS.
uint32_t dense_groups(uint64_t rows, uint64_t cols) {
    if (cols > 2048) return (uint32_t) rows;
    const uint64_t per = 4 * std::min<uint64_t>(8, std::max<uint64_t>(1, rows / 1024));   // dense_rpw
    return (uint32_t) ((rows + per - 1) / per);
}
uint32_t dense_lds(uint64_t cols, uint32_t m) { return cols > 2048 ? 128u : (uint32_t) (m * cols * 4); }

// Workgroups of a kernel that loops over its work (the head): a few per compute unit of the MI355X's 256.
uint32_t persistent_groups() {
    static const uint32_t n = [] {
        const char* e = std::getenv("SHADOWZERO_HEAD_GROUPS");
        const int v = e ? std::atoi(e) : 0;
        return (uint32_t) (v > 0 ? v : 768);
    }();
    return n;
}

// Partial sums an EXL3 product leaves per output: one wave takes 128 inputs of a 128-output block, the four waves of a
// workgroup add theirs up.
uint32_t exl3_ksplit(uint32_t in_f) { return (in_f / 128 + 3) / 4; }

static int check_exl3_shape(uint64_t in_f, uint64_t out_f) {
    if (in_f == 0 || out_f == 0 || in_f % 128 || out_f % 128) return fail("EXL3 projections need in and out to be multiples of 128");
    return 0;
}

// ---- device scratch that grows on demand (backend.rs:42-52) ---------------------------------------------------------
struct DevBuf {
    uint64_t ptr = 0, bytes = 0;
    int need(uint64_t n) {
        if (bytes >= n) return 0;
        if (ptr) sz_free(ptr);
        ptr = 0;
        bytes = 0;
        if (sz_malloc(&ptr, n)) return 1;
        bytes = n;
        return 0;
    }
    ~DevBuf() {
        if (ptr && initialized()) sz_free(ptr);
    }
};

// ---- one product y_j = W x_j, j < m, on device pointers ---------------------------------------------------------------
// EXL3 workspace layout: u64 wtab[ng] | u32 gtab[17 ng] (16-byte aligned) | f32 part[ng * ks * 4 * rows]
static uint64_t align16(uint64_t v) { return (v + 15) & ~15ull; }

static uint64_t cols_scratch_bytes(const Format& f, uint64_t cols, uint64_t rows, uint32_t m) {
    if (!f.exl3) return 0;
    const uint64_t ng = (m + 3) / 4;
    return align16(ng * 8) + align16(ng * 17 * 4) + ng * exl3_ksplit((uint32_t) cols) * 4 * rows * 4;
}

int matvec_cols_dev(int ty, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys, uint32_t m,
                           uint64_t scratch, uint64_t scratch_bytes, uint64_t stream) {
    Format f;
    std::string tag;
    if (!format_of(ty, f, tag)) return fail("no matvec kernel for ggml type " + std::to_string(ty));
    if (m == 0 || m > 8) return fail("matvec_cols takes 1..8 inputs");
    if (xs < cols || ys < rows) return fail("matvec_cols: row strides shorter than the rows");
    if (cols >> 31 || rows >> 31) return fail("matvec_cols: shape too large");
    if (f.exl3) {
        if (check_exl3_shape(cols, rows)) return 1;
        if (xs % 4 || (x & 15)) return fail("matvec_cols: inputs must be 16-byte aligned");
        const uint32_t ng = (m + 3) / 4, ks = exl3_ksplit((uint32_t) cols);
        if (scratch_bytes < cols_scratch_bytes(f, cols, rows, m) || !scratch) return fail("matvec_cols: workspace too small for EXL3");
        const uint64_t wtab = scratch, gtab = scratch + align16(ng * 8), part = gtab + align16(ng * 17 * 4);
        const sz_arg a0[] = {P(wtab), P(gtab), U64(w), U32(m)};
        if (launch("cols_plan", 1, 1, 1, 64, 0, stream, a0)) return 1;
        const std::string kn = "matvec_grouped_" + tag;
        const sz_arg a1[] = {P(wtab), P(gtab), P(x), U32(xs), P(part), U32((uint32_t) cols), U32((uint32_t) rows)};
        if (launch(kn.c_str(), (uint32_t) rows / 128, ng, ks, 256, 0, stream, a1)) return 1;
        const sz_arg a2[] = {P(part), P(wtab), P(gtab), P(y), U32(ys), U32((uint32_t) cols), U32((uint32_t) rows)};
        return launch("exl3_finish_rows", (uint32_t) rows / 128, ng, 1, 64, 0, stream, a2);
    }
    if (f.dense) {
        if (rows == 0) return 0;
        if (cols % 4 || (x & 15) || xs % 4 || (w & (4 * f.bb - 1))) return fail("matvec_cols: unquantized matrices need columns in fours and aligned rows");
        const std::string kn = "matvec_cols_" + tag;
        const sz_arg a[] = {P(w), P(x), U32(xs), P(y), U32(ys), U32((uint32_t) rows), U32((uint32_t) cols), U32(m)};
        return launch(kn.c_str(), dense_groups(rows, cols), 1, 1, 256, dense_lds(cols, m), stream, a);
    }
    if (cols % f.qk) return fail("matvec_cols: columns are not whole blocks");
    // fewer rows a workgroup where the launch would otherwise have under about 512 workgroups (two a CU)
    const uint32_t rpb = rows_per_block(f, (uint32_t) cols, (uint32_t) std::max<uint64_t>(1, rows * ((m + 3) / 4) / 512));
    if (rpb == 0 || (x & 15) || xs % 4) {
        // any shape: the one-weight-at-a-time kernel, an input at a time
        const std::string kn = "matvec_" + tag;
        for (uint32_t j = 0; j < m; j++) {
            const sz_arg a[] = {P(w), P(x + (uint64_t) j * xs * 4), P(y + (uint64_t) j * ys * 4), U32((uint32_t) rows), U32((uint32_t) cols)};
            if (launch(kn.c_str(), ((uint32_t) rows + 3) / 4, 1, 1, 256, 0, stream, a)) return 1;
        }
        return 0;
    }
    const uint32_t rb = (uint32_t) cols / f.qk * f.bb;
    const std::string kn = "matvec_cols_" + tag;
    const sz_arg a[] = {P(w), P(x), U32(xs), P(y), U32(ys), U32((uint32_t) rows), U32((uint32_t) cols), U32(m), U32(rpb)};
    return launch(kn.c_str(), ((uint32_t) rows + rpb - 1) / rpb, (m + 3) / 4, 1, 256, rpb * rb + 32, stream, a);
}

}   // namespace sz

using namespace sz;

// ---- B1: Backend ----------------------------------------------------------------------------------------------------
// Pinned host memory that the device reads and writes directly (grown on demand, freed with its owner).
struct PinnedBuf {
    void* ptr = nullptr;
    uint64_t bytes = 0;
    int need(uint64_t n) {
        if (bytes >= n) return 0;
        if (ptr) hip().hipHostFree(ptr);
        ptr = nullptr;
        bytes = 0;
        if (hip_check(hip().hipHostMalloc(&ptr, n, 0), "hipHostMalloc")) return 1;
        bytes = n;
        return 0;
    }
    ~PinnedBuf() {
        if (ptr) hip().hipHostFree(ptr);
    }
};

struct sz_backend {
    uint64_t budget = 0, resident_bytes = 0, uploads = 0;
    std::unordered_map<std::string, DevBuf> resident;
    DevBuf w, x, scratch;
    PinnedBuf hx, hy;   // the call's input on its way to the device, and its output, which the kernel writes here itself
};

extern "C" {

sz_backend* sz_backend_new(uint64_t budget) {
    clear_error();
    if (ensure_init()) return nullptr;
    sz_backend* b = new sz_backend();
    b->budget = budget;
    return b;
}
void sz_backend_free(sz_backend* b) { delete b; }
uint64_t sz_backend_resident_bytes(const sz_backend* b) { return b->resident_bytes; }
uint64_t sz_backend_uploads(const sz_backend* b) { return b->uploads; }

int32_t sz_matvec(sz_backend* b, int32_t ty, uint64_t cols, uint64_t rows, const void* bytes, uint64_t nbytes, const char* key, const float* x,
                  float* y) {
    clear_error();
    if (!b) return fail("sz_matvec: null backend");
    Format f;
    std::string tag;
    if (!format_of(ty, f, tag)) return fail("no matvec kernel for ggml type " + std::to_string(ty));   // the reference panics here (backend.rs:60)
    if (!f.exl3 && (cols == 0 || cols % f.qk)) return fail("sz_matvec: columns are not whole blocks");
    if (!f.exl3 && rows == 0) rows = nbytes / (cols / f.qk * f.bb);
    if (f.exl3 && check_exl3_shape(cols, rows)) return 1;
    if (matrix_bytes(f, cols, rows) != nbytes) return fail("sz_matvec: " + std::to_string(nbytes) + " bytes for " + std::to_string(rows) + " x " + std::to_string(cols) + " of " + tag);
    uint64_t wp = 0;
    if (key) {
        auto it = b->resident.find(key);
        if (it != b->resident.end()) {
            if (it->second.bytes < nbytes) return fail(std::string("sz_matvec: resident tensor ") + key + " is smaller than the bytes given");
            wp = it->second.ptr;
        } else if (b->resident_bytes + nbytes <= b->budget) {
            DevBuf& d = b->resident[key];
            if (d.need(nbytes) || sz_upload(d.ptr, bytes, nbytes)) {
                b->resident.erase(key);
                return 1;
            }
            b->resident_bytes += nbytes;
            b->uploads++;
            wp = d.ptr;
        }
    }
    if (!wp) {
        if (b->w.need(nbytes) || sz_upload(b->w.ptr, bytes, nbytes)) return 1;
        b->uploads++;
        wp = b->w.ptr;
    }
    // x goes through pinned memory with an asynchronous copy and y is written into pinned memory by the kernel itself: the call
    // waits once, for the stream, instead of once a blocking copy each way (31 -> 20 us a call for a resident 1024 x 2048 matrix)
    if (b->x.need(cols * 4) || b->hx.need(cols * 4) || b->hy.need(rows * 4)) return 1;
    std::memcpy(b->hx.ptr, x, cols * 4);
    if (hip_check(hip().hipMemcpyHtoDAsync((void*) b->x.ptr, b->hx.ptr, cols * 4, nullptr), "hipMemcpyHtoDAsync")) return 1;
    const uint64_t sb = cols_scratch_bytes(f, cols, rows, 1);
    if (sb && b->scratch.need(sb)) return 1;
    if (matvec_cols_dev(ty, wp, cols, rows, b->x.ptr, (uint32_t) cols, (uint64_t) b->hy.ptr, (uint32_t) rows, 1, b->scratch.ptr, b->scratch.bytes, 0)) return 1;
    if (sz_stream_synchronize(0)) return 1;   // synchronous, as the reference's backend: waits for the kernels
    std::memcpy(y, b->hy.ptr, rows * 4);
    return 0;
}

// ---- B4: device entry points ------------------------------------------------------------------------------------------
int32_t sz_dequantize(int32_t ty, uint64_t w, uint64_t out, uint64_t cols, uint64_t rows, uint64_t stream) {
    clear_error();
    Format f;
    std::string tag;
    if (!format_of(ty, f, tag)) return fail("no dequantizer for ggml type " + std::to_string(ty));
    if (f.exl3) {
        if (check_exl3_shape(cols, rows)) return 1;
        const std::string kn = std::string(f.half ? "exl3_decode_h" : "exl3_decode_") + std::to_string(f.bits);
        const sz_arg a[] = {P(w), P(out), U32((uint32_t) cols), U32((uint32_t) rows)};
        return launch(kn.c_str(), (uint32_t) rows / 128, (uint32_t) cols / 16, 1, 64, 0, stream, a);
    }
    if (f.dense) return fail("sz_dequantize: an unquantized matrix has nothing to dequantize");
    if (cols % f.qk) return fail("sz_dequantize: columns are not whole blocks");
    const uint64_t n = cols * rows;
    if (n == 0) return 0;
    const std::string kn = "dequant_" + tag;
    const sz_arg a[] = {P(w), P(out), U64(n)};
    return launch(kn.c_str(), (uint32_t) ((n + 255) / 256), 1, 1, 256, 0, stream, a);
}

int32_t sz_exl3_codebook(uint64_t out, uint64_t stream) {
    clear_error();
    const sz_arg a[] = {P(out), U32(65536)};
    return launch("exl3_codebook", 256, 1, 1, 256, 0, stream, a);
}

uint64_t sz_matvec_cols_scratch(int32_t ty, uint64_t cols, uint64_t rows, uint32_t m) {
    Format f;
    std::string tag;
    if (!format_of(ty, f, tag)) return 0;
    return cols_scratch_bytes(f, cols, rows, m);
}

int32_t sz_matvec_cols(int32_t ty, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys, uint32_t m,
                       uint64_t scratch, uint64_t scratch_bytes, uint64_t stream) {
    clear_error();
    return matvec_cols_dev(ty, w, cols, rows, x, xs, y, ys, m, scratch, scratch_bytes, stream);
}

}   // extern "C"

// One matrix of a matvec_cols_multi launch (DenseJob of kernels/matvec.hip).
struct DenseJob {
    uint64_t w, y;
    uint32_t ys, rows, type, first, act;
    float div;
};
static_assert(sizeof(DenseJob) == 40, "the kernel reads this layout");

// ---- B2: the session ----------------------------------------------------------------------------------------------------
struct SzLayer {
    int type = 0, shared_type = 0;
    uint64_t experts = 0, stride = 0, shared = 0;
    uint64_t gap = 0; // bytes between an expert's projections (0: the reference's contiguous [gate|up|down])
    DevBuf eaddr;     // u64[3 * ne] then u64[3] for the shared expert
    DevBuf jobs;      // the router launch's job table (set_router)
    uint32_t router_groups = 0;
    bool set = false;
};

struct SzGraphKey {
    uint64_t v[10];
    bool operator<(const SzGraphKey& o) const { return std::memcmp(v, o.v, sizeof v) < 0; }
};

struct sz_session {
    sz_session_config cfg{};
    std::vector<SzLayer> layers;
    int head_type = 0;
    uint64_t head_w = 0;
    // batch buffers (session.rs `bb`): the plan, the expert products, the split-k partials, the head's scratch
    DevBuf plan, eg, act, eo, part, dn, head_part, logits, topv, topi, ids;
    DevBuf plans;                 // a plan a layer for the rounds that route every layer up front (sz_verify_round)
    uint32_t plan_stride = 0;
    DevBuf head_xa, head_inv;   // an EXL3 head's rotated inputs as f16 high and low parts (16 rows of 128 a 128-block), and the tokens' scales
    DevBuf rl, sgl;   // the router's outputs for a batch: f32[max_rows][n_expert], f32[max_rows]
    // the optional 2-bit screen of an EXL3 head (HeadProxy of session.rs:428-441): k_blk = 0 is off
    struct {
        uint32_t k_blk = 0;
        DevBuf w_q2, w_sc, xq, x_sc, x_corr, bmax, seen, sel, logits;
    } hp;
    struct {
        DevBuf xq, xd, tidx, w, cnt, offs, list, items, hq, hd, eo, gup, arows, ainv;
    } pf;   // the prefill chunk's buffers, grown on demand
    void* top_host = nullptr;  // pinned host memory the top-64 merge writes to directly (8 rows of 128 words): no copy back
    bool last_fused = false;   // the last layer call left its routing in the fused layout [tidx | w | cnt]
    // how an EXL3 layer at a whole bit rate multiplies (sz_session_set_expert_mode): 0 the exact kernels, a weight at a time on
    // the vector unit; 1 the matrix cores with the codebook's own f16 values; 2 the matrix cores with the linearised codebook
    int expert_mode = 0;
    DevBuf plan2;              // a round's layers alternate between two plans: the sum of a layer rides the next layer's first launch, which writes that layer's routing
    uint64_t last_plan = 0;    // the plan the last layer call left its routing in
    std::map<SzGraphKey, uint64_t> graphs;
    // plan offsets for the largest batch
    uint32_t GT_max = 0;
    bool use_graph = true;
};

namespace {

struct PlanLayout {
    uint32_t G, nsh, GT, R, a0, r0, w_off, counts_off, tidx_off, bytes;
};

PlanLayout plan_layout(uint32_t m, uint32_t k) {
    PlanLayout p{};
    p.G = m * k;
    p.nsh = (m + 3) / 4;
    p.GT = p.G + p.nsh;
    p.R = p.G + m;                       // rows of the expert products: the pairs, then the shared expert's m rows
    p.a0 = 0;
    p.r0 = (uint32_t) align16(p.a0 + 3 * p.GT * 8);
    p.w_off = (uint32_t) align16(p.r0 + 3 * p.GT * 17 * 4);
    p.counts_off = (uint32_t) align16(p.w_off + m * k * 4);
    p.tidx_off = (uint32_t) align16(p.counts_off + m * 4);
    p.bytes = (uint32_t) align16(p.tidx_off + m * k * 4);
    return p;
}

// The matrix-core EXL3 layer's plan behind [tidx | w | cnt] (verify_plan_exl3 in kernels/exl3.hip): byte offset of the item
// list, item slots (one a pair plus the shared expert's, an even number), bytes of the whole.
struct MmaPlan {
    uint32_t ioff, slots, bytes;
};
MmaPlan mma_plan(uint32_t m, uint32_t k) {
    MmaPlan p{};
    p.ioff = (uint32_t) align16(2ull * m * k * 4 + m * 4);
    p.slots = (m * k + 3) & ~1u;   // at least one more than the most items there can be: the last slot is never an item
    p.bytes = p.ioff + 16 + p.slots * 32;
    return p;
}
// Dynamic LDS of its two product launches: EXL3_MMA_LDS_WORDS there (a 4-row ring, the A rows and the scales of 4 waves).
uint32_t mma_lds_bytes(int bits, uint32_t nmax) {
    const uint32_t stride = (bits == 3 || bits == 4) ? 4 : (uint32_t) bits;
    const uint32_t ring = 4 * 64 * stride;
    return 4 * (4 * (ring + nmax * 128 + 64 + 16) + 64);
}

// The rank-order sum of an EXL3 layer that has not been launched yet: inside sz_verify_round it rides the first launch of
// the layer after it (whose routing goes to the session's other plan buffer), and the last layer's gets a launch of its own.
struct PendingSum {
    bool active = false;
    uint64_t plan = 0, sgl = 0, y = 0;
    bool shared = false;
    // the round's routing launch (verify_route_layers) has filled a plan a layer, `plan_stride` apart from `plans` on: the
    // exact EXL3 launches of those layers get no logits and read their plan instead of redoing the selection
    uint64_t plans = 0;
    uint32_t plan_stride = 0;
};

int launch_pending_sum(sz_session* s, PendingSum& ps, uint32_t m, uint64_t stream) {
    if (!ps.active) return 0;
    const sz_session_config& c = s->cfg;
    ps.active = false;
    const sz_arg a[] = {P(s->dn.ptr), U64(0), U64(0), U64(ps.shared ? 1 : 0), U32(0), P(ps.plan), P(ps.sgl), P(ps.y),
                        U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(0)};
    return launch("verify_combine_exl3", c.hidden / 128, m, 1, 128, 0, stream, a);
}

int moe_layer(sz_session* s, uint32_t l, uint32_t m, uint64_t u, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t stream, PendingSum* ride = nullptr) {
    const sz_session_config& c = s->cfg;
    if (l >= s->layers.size() || !s->layers[l].set) return fail("sz_moe_layer_verify: layer " + std::to_string(l) + " has no experts set");
    if (m == 0 || m > c.max_rows) return fail("sz_moe_layer_verify: " + std::to_string(m) + " rows (1.." + std::to_string(c.max_rows) + ")");
    if ((u & 15) || (y & 15)) return fail("sz_moe_layer_verify: activations must be 16-byte aligned");
    SzLayer& L = s->layers[l];
    Format f;
    std::string tag;
    if (!format_of(L.type, f, tag)) return fail("layer type " + std::to_string(L.type) + " has no kernels");
    const bool shared = L.shared != 0;
    if (shared && L.shared_type != L.type) return fail("the shared expert must have the routed experts' type (layer " + std::to_string(l) + ")");
    const PlanLayout p = plan_layout(m, c.top_k);
    // a layer whose sum may ride the next launch takes the plan buffer the pending sum is not reading; a layer routed by the
    // round's routing launch has a plan of its own
    const bool f16x = s->expert_mode == 3 && f.exl3 && !f.half;   // the exact launches with f16 inputs and two products an instruction
    const bool routed = ride && ride->plans && f.exl3 && (s->expert_mode == 0 || s->expert_mode == 3);
    const uint64_t plan = routed ? ride->plans + (uint64_t) l * ride->plan_stride
                                 : (ride && ride->active && ride->plan == s->plan.ptr) ? s->plan2.ptr : s->plan.ptr;
    s->last_plan = plan;
    const uint64_t addr = plan + p.a0, rec = plan + p.r0, wts = plan + p.w_off, cnt = plan + p.counts_off;
    const uint64_t addr_d = addr + 2ull * p.GT * 8, rec_d = rec + 2ull * p.GT * 17 * 4;
    const std::string kn = "matvec_grouped_" + tag;
    if (ride && ride->active && !f.exl3 && launch_pending_sum(s, *ride, m, stream)) return 1;   // only an EXL3 layer's first launch carries a sum
    // the sum of the layer before, if it rides this layer's first launch: the workgroups it adds, its arguments
    const bool carry = f.exl3 && ride && ride->active;
    const uint32_t carry_groups = carry ? c.hidden / 128 * m : 0;
    const uint64_t c_plan = carry ? ride->plan : 0, c_sgl = carry ? ride->sgl : 0, c_y = carry ? ride->y : 0;
    const uint32_t c_mode = carry ? (ride->shared ? 2 : 1) : 0;
    // this layer's own sum: left for the next launch to carry when the caller takes care of it (launch 2 must have finished the blocks)
    auto sum = [&](uint32_t zs_d, uint64_t part) -> int {
        if (ride) ride->active = false;
        s->last_fused = true;
        if (ride && zs_d == 1) {
            ride->active = true;
            ride->plan = plan;
            ride->sgl = sgl;
            ride->y = y;
            ride->shared = shared;
            return 0;
        }
        const sz_arg a[] = {P(s->dn.ptr), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(plan), P(sgl), P(y),
                            U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(zs_d == 1 ? 0 : zs_d)};
        return launch("verify_combine_exl3", c.hidden / 128, m, 1, zs_d == 1 ? 128 : 1024, 0, stream, a);   // zs_d == 1: launch 2 finished the blocks
    };
    if (f.exl3 && !f.half && (s->expert_mode == 1 || s->expert_mode == 2)) {
        // the matrix-core layer: a plan of the batch's distinct experts, then gate/up and down with an item's tokens on the rows
        // of the matrix instruction, then the rank-order sum (kernels/exl3.hip, "the verify layer on the matrix cores")
        const MmaPlan mp = mma_plan(m, c.top_k);
        const uint32_t zs_gu = (c.hidden / 128 + 3) / 4, zs_d = exl3_ksplit(c.ff);
        const uint64_t part = matrix_bytes(f, c.hidden, c.ff) + L.gap;   // from one projection of an expert to the next
        if (part >> 32) return fail("sz_moe_layer_verify: a projection of 4 GiB or more");
        const uint32_t nmax = m > 4 ? 8 : 4;
        const uint32_t lds = mma_lds_bytes(f.bits, nmax);
        const std::string variant = std::string(s->expert_mode == 2 ? "lin" : "mma") + (nmax == 8 ? "w" : "");
        const std::string k1 = "verify_gate_up_" + variant + "_" + tag, k2 = "verify_down_" + variant + "_" + tag;
        {
            const sz_arg a[] = {P(rl), P(plan), U32(mp.ioff), U32(c.n_expert), U32(c.top_k), U32(m), U32(shared ? 1 : 0), U32(c.hidden),
                                P(s->dn.ptr), P(c_plan), P(c_sgl), P(c_y), U32(c_mode)};
            if (launch("verify_plan_exl3", 1 + carry_groups, 1, 1, 64 * m, 0, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(u), P(plan), U32(mp.ioff), P(s->part.ptr),
                                U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff)};
            if (launch(k1.c_str(), c.ff / 128, 2 * mp.slots, zs_gu, 256, lds, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(plan), U32(mp.ioff), P(s->part.ptr), P(s->dn.ptr),
                                U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(zs_gu)};
            if (launch(k2.c_str(), c.hidden / 128, mp.slots, zs_d, 256, lds, stream, a)) return 1;
        }
        return sum(zs_d, part);
    } else if (f.exl3) {
        // the fused layer: three launches, the work items are the (token, rank) pairs themselves, no plan.  A wave of
        // launch 1 takes one 128-block of the input, 4 waves a workgroup (EXL3_GU_WAVES, EXL3_VERIFY_NB in kernels/exl3.hip).
        const uint32_t S = p.G + m, zs_gu = (c.hidden / 128 + 3) / 4, zs_d = exl3_ksplit(c.ff);
        const uint64_t part = matrix_bytes(f, c.hidden, c.ff) + L.gap;   // from one projection of an expert to the next
        if (part >> 32) return fail("sz_moe_layer_verify: a projection of 4 GiB or more");
        const std::string ftag = f16x ? "exl3f_" + std::to_string(f.bits) : tag;
        const std::string k1 = "verify_gate_up_" + ftag, k2 = "verify_down_" + ftag;
        {
            const uint32_t gx = c.ff / 128, extra = (carry_groups + gx * zs_gu - 1) / (gx * zs_gu);   // rows of the grid for a riding sum
            const sz_arg a[] = {P(routed ? 0 : rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(u), P(plan), P(s->part.ptr),
                                U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), P(s->dn.ptr), P(c_plan), P(c_sgl), P(c_y), U32(c_mode)};
            if (launch(k1.c_str(), gx, 2 * S + extra, zs_gu, 256, 0, stream, a)) return 1;   // 4 waves of one 128-block each: EXL3_GU_WAVES, EXL3_VERIFY_NB
        }
        {
            const sz_arg a[] = {P(routed ? 0 : rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(plan), P(s->part.ptr), P(s->dn.ptr),
                                U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(zs_gu)};
            if (launch(k2.c_str(), c.hidden / 128, S, zs_d, 256, 0, stream, a)) return 1;
        }
        return sum(zs_d, part);
    } else if (!std::getenv("SHADOWZERO_GGUF_PLANNED") && c.ff <= 4096) {
        // the pair form, as the EXL3 layer: routing inside launch 1, SwiGLU inside launch 2, no plan
        const uint32_t S = p.G + m;
        // (one row has few pairs to hand out: 16 and 32 rows a workgroup fill the chip better than 32 and 64, which win from two rows on: measured)
        const uint32_t rpb_gu = rows_per_block(f, c.hidden, m == 1 ? 16 : 32, m == 1 ? 16384 : 32768);
        const uint32_t rpb_d = rows_per_block(f, c.ff, m == 1 ? 32 : 64);
        if (!rpb_gu || !rpb_d) return fail("sz_moe_layer_verify: no kernel for hidden = " + std::to_string(c.hidden) + ", ff = " + std::to_string(c.ff));
        const uint64_t part = matrix_bytes(f, c.hidden, c.ff) + L.gap;   // from one projection of an expert to the next
        if (part >> 32) return fail("sz_moe_layer_verify: a projection of 4 GiB or more");
        const uint32_t rb_gu = c.hidden / f.qk * f.bb, rb_d = c.ff / f.qk * f.bb;
        // One token: two launches.  Launch 1 hands over act = silu(gate) * up and the routing weights, launch 2 owns a row chunk
        // for all of the token's experts and adds them up itself (SHADOWZERO_GGUF_THREE_LAUNCH=1 keeps the general form).
        const bool three = std::getenv("SHADOWZERO_GGUF_THREE_LAUNCH") != nullptr;
        const uint32_t uh = c.hidden / 32, uf = c.ff / 32;
        if (m == 1 && !three && c.hidden % 32 == 0 && c.ff % 32 == 0 && uh <= 64 && 64 % uh == 0 && uf <= 64 && 64 % uf == 0 && c.top_k <= 16) {
            const uint32_t rp = 8, rd = std::max(4u, 64 / uf);
            const uint32_t rs_gu = (rp * rb_gu + 31) / 16 * 16, rs_d = (rd * rb_d + 31) / 16 * 16;
            const uint32_t Sd = c.top_k + (shared ? 1 : 0);
            if (c.ff % rp == 0 && c.hidden % rd == 0 && 2 * rs_gu <= 16384 && Sd * rs_d <= 16384 && Sd * c.ff <= 8192) {
                const std::string d1 = "decode_gate_up_" + tag, d2 = "decode_down_combine_" + tag;
                {
                    const sz_arg a[] = {P(rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(u), P(plan), P(s->eg.ptr),
                                        U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(rp)};
                    if (launch(d1.c_str(), c.ff / rp, S, 1, 512, 2 * rs_gu, stream, a)) return 1;   // 8 waves: a gate row and an up row each at hidden 2048
                }
                s->last_fused = true;
                const sz_arg a[] = {U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(plan), P(s->eg.ptr), P(sgl), P(y),
                                    U32(c.top_k), U32(c.hidden), U32(c.ff), U32(rd)};
                return launch(d2.c_str(), c.hidden / rd, 1, 1, 64 * std::min(16u, std::max(4u, Sd)), Sd * rs_d + Sd * uf * 144, stream, a);   // a wave a pair
            }
        }
        const std::string k1 = "verify_gate_up_" + tag, k2 = "verify_down_" + tag;
        {
            const sz_arg a[] = {P(rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(u), P(plan), P(s->eg.ptr),
                                U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(rpb_gu)};
            if (launch(k1.c_str(), (c.ff + rpb_gu - 1) / rpb_gu, 2 * S, 1, 256, rpb_gu * rb_gu + 32, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(rl), U64(L.experts), U64(L.stride), U64(L.shared), U32((uint32_t) part), P(plan), P(s->eg.ptr), P(s->eo.ptr),
                                U32(c.n_expert), U32(c.top_k), U32(m), U32(c.hidden), U32(c.ff), U32(rpb_d)};
            if (launch(k2.c_str(), (c.hidden + rpb_d - 1) / rpb_d, S, 1, 256, rpb_d * rb_d + 32, stream, a)) return 1;
        }
        s->last_fused = true;
        const uint64_t G4 = (uint64_t) p.G * 4;
        const sz_arg a[] = {P(y), P(s->eo.ptr), P(plan + G4), P(shared ? s->eo.ptr + (uint64_t) p.G * c.hidden * 4 : 0), P(sgl), P(plan + 2 * G4),
                            U32(c.hidden), U32(c.top_k)};
        return launch("moe_combine_qwen_rows", (c.hidden + 255) / 256, m, 1, 256, 0, stream, a);
    } else {
        {
            const sz_arg a[] = {P(rl), P(L.eaddr.ptr), P(plan), U32(c.n_expert), U32(c.top_k), U32(m), U32(p.G), U32(p.R), U32(p.a0), U32(p.r0),
                                U32(p.w_off), U32(p.counts_off), U32(p.tidx_off), P(shared ? L.eaddr.ptr + 3ull * c.n_expert * 8 : 0)};
            if (launch("route_plan_res_small", 1, 1, 1, 256, 0, stream, a)) return 1;
        }
        s->last_fused = false;
        const uint32_t rpb_gu = rows_per_block(f, c.hidden, std::max<uint32_t>(1, c.ff * 2 * p.GT / 512));
        const uint32_t rpb_d = rows_per_block(f, c.ff, std::max<uint32_t>(1, c.hidden * p.GT / 512));
        if (!rpb_gu || !rpb_d) return fail("this hidden / ff shape is not supported by the grouped " + tag + " kernels");
        const uint32_t rb_gu = c.hidden / f.qk * f.bb, rb_d = c.ff / f.qk * f.bb;
        {
            const sz_arg a[] = {P(addr), P(rec), P(u), U32(c.hidden), P(s->eg.ptr), U32(c.ff), U32(c.ff), U32(c.hidden), U32(rpb_gu)};
            if (launch(kn.c_str(), (c.ff + rpb_gu - 1) / rpb_gu, 2 * p.GT, 1, 256, rpb_gu * rb_gu + 32, stream, a)) return 1;
        }
        {
            const uint32_t n = p.R * c.ff;
            const sz_arg a[] = {P(s->eg.ptr), P(s->eg.ptr + (uint64_t) p.R * c.ff * 4), P(s->act.ptr), U32(n)};
            if (launch("swiglu", (n + 255) / 256, 1, 1, 256, 0, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(addr_d), P(rec_d), P(s->act.ptr), U32(c.ff), P(s->eo.ptr), U32(c.hidden), U32(c.hidden), U32(c.ff), U32(rpb_d)};
            if (launch(kn.c_str(), (c.hidden + rpb_d - 1) / rpb_d, p.GT, 1, 256, rpb_d * rb_d + 32, stream, a)) return 1;
        }
    }
    const sz_arg a[] = {P(y), P(s->eo.ptr), P(wts), P(shared ? s->eo.ptr + (uint64_t) p.G * c.hidden * 4 : 0), P(sgl), P(cnt), U32(c.hidden), U32(c.top_k)};
    return launch("moe_combine_qwen_rows", (c.hidden + 255) / 256, m, 1, 256, 0, stream, a);
}

// The head for rows [j0, j0 + n) with the arg-max fused in; logits (0: not written) has rows c.vocab apart.
int head_argmax_rows(sz_session* s, uint32_t n, uint64_t u, uint64_t logits, uint64_t ids, uint64_t stream) {
    const sz_session_config& c = s->cfg;
    Format f;
    std::string tag;
    format_of(s->head_type, f, tag);
    const uint32_t rpb = rows_per_block(f, c.hidden);
    if (!rpb) return fail("the head kernel does not support hidden = " + std::to_string(c.hidden));
    const uint32_t rb = c.hidden / 32 * 34, nchunks = (c.vocab + rpb - 1) / rpb;
    const uint32_t nparts = std::min<uint32_t>(nchunks, persistent_groups());
    const sz_arg a[] = {P(s->head_w), P(u), U32(c.hidden), P(logits), U32(c.vocab), P(s->head_part.ptr), U32(c.vocab), U32(c.hidden), U32(n), U32(rpb)};
    if (launch("head_q8_0_argmax", nparts, 1, 1, 256, rpb * rb + 32 + rpb * 16, stream, a)) return 1;
    const sz_arg b[] = {P(s->head_part.ptr), U32(nparts), U32(4), P(ids), P(0)};
    return launch("argmax_merge_parts", n, 1, 1, 256, 0, stream, b);
}

// The end of a head pass: the rows' arg-max ids out of the partial maxima; with `accept` set (a verify round), the greedy
// acceptance of the drafts in the same launch.
struct Accept {
    uint64_t drafts = 0, out = 0;
};
int merge_parts(sz_session* s, uint32_t nparts, uint32_t ts, uint32_t m, uint64_t ids, const Accept* accept, uint64_t stream) {
    if (accept) {
        const sz_arg a[] = {P(s->head_part.ptr), U32(nparts), U32(ts), P(ids), U32(m), P(accept->drafts), U32(m - 1), P(accept->out)};
        return launch("argmax_merge_accept", 1, 1, 1, 1024, 0, stream, a);
    }
    const sz_arg b[] = {P(s->head_part.ptr), U32(nparts), U32(ts), P(ids), P(0)};
    return launch("argmax_merge_parts", m, 1, 1, 256, 0, stream, b);
}

// The matrix-core head: all m <= 8 rows in one pass over the matrix.  The number of waves a workgroup (each owns at most
// 512 columns of a row): 4 up to 2048 columns, 6 up to 3072, 8 up to 4096; 0: the shape goes to the scalar kernel.
uint32_t head_mfma_waves(const sz_session* s) {
    static const bool off = std::getenv("SHADOWZERO_HEAD_SCALAR") != nullptr;
    const sz_session_config& c = s->cfg;
    if (off || s->head_type != SZ_TYPE_Q8_0 || (s->head_w & 15) != 0 || c.vocab < 16) return 0;
    if (c.hidden % 256 == 0 && c.hidden <= 2048) return 4;
    if (c.hidden % 192 == 0 && c.hidden <= 3072) return 6;
    if (c.hidden % 256 == 0 && c.hidden <= 4096) return 8;
    return 0;
}
bool head_mfma_ok(const sz_session* s) { return head_mfma_waves(s) != 0; }

int head_argmax_mfma(sz_session* s, uint32_t m, uint64_t u, uint64_t logits, uint64_t ids, uint64_t stream, const Accept* accept = nullptr) {
    const sz_session_config& c = s->cfg;
    const uint32_t waves = head_mfma_waves(s);
    const uint32_t tiles = (c.vocab + 15) / 16;
    const uint32_t nparts = std::min<uint32_t>(tiles, waves == 4 ? 512 : 256);       // two workgroups a CU (70 KB of LDS each), one for the wider rows
    const sz_arg a[] = {P(s->head_w), P(u), U32(c.hidden), P(logits), U32(c.vocab), P(s->head_part.ptr), U32(c.vocab), U32(c.hidden), U32(m)};
    const char* name = waves == 4 ? "head_q8_0_argmax_mfma" : waves == 6 ? "head_q8_0_argmax_mfma_w6" : "head_q8_0_argmax_mfma_w8";
    static const bool four_waves = std::getenv("SHADOWZERO_HEAD_FOUR_WAVES") != nullptr;   // the general form at 2048 columns too, for comparisons
    if (waves == 4 && c.hidden == 2048 && !four_waves) {
        // rows of exactly 2048 columns: 8 waves of 256 columns each on the same two tiles of LDS, no per-block checks
        if (launch("head_q8_0_argmax_mfma_n8", nparts, 1, 1, 512, 0, stream, a)) return 1;
        return merge_parts(s, nparts, 8, m, ids, accept, stream);
    }
    if (launch(name, nparts, 1, 1, 64 * waves, 0, stream, a)) return 1;
    return merge_parts(s, nparts, 8, m, ids, accept, stream);
}

bool head_is_exl3(const sz_session* s) { return s->head_type >= 1021 && s->head_type <= 1028; }

// LDS of a workgroup of head_exl3_K for m rows: the four waves' 4-row rings (static; a row is 64 lanes x 4 words at K = 3 and
// 4, x K words otherwise) and the A rows, 4 KiB for every 512 inputs and every two rows (dynamic).  A compute unit of the
// MI355X has 160 KiB.
const uint32_t CU_LDS_BYTES = 160 * 1024;
uint32_t exl3_head_lds_dynamic(uint32_t hidden, uint32_t m) { return 4 * ((hidden / 128 + 3) / 4) * ((m + 1) / 2) * 1024; }
uint32_t exl3_head_lds(uint32_t bits, uint32_t hidden, uint32_t m) {
    const uint32_t stride = (bits == 3 || bits == 4) ? 4 : bits;
    return 4 * (4 * 64 * stride) * 4 + exl3_head_lds_dynamic(hidden, m);
}

int head_check(sz_session* s, uint32_t m, uint64_t u, const char* who) {
    if (!s->head_w) return fail(std::string(who) + ": no head set");
    if (m == 0 || m > s->cfg.max_rows) return fail(std::string(who) + ": " + std::to_string(m) + " rows");
    if (u & 15) return fail(std::string(who) + ": activations must be 16-byte aligned");
    if (head_is_exl3(s) && exl3_head_lds((uint32_t) s->head_type - 1020, s->cfg.hidden, m) > CU_LDS_BYTES)
        return fail(std::string(who) + ": an EXL3 head of hidden " + std::to_string(s->cfg.hidden) + " at " + std::to_string(s->head_type - 1020) + " bits takes " +
                    std::to_string(exl3_head_lds((uint32_t) s->head_type - 1020, s->cfg.hidden, m)) + " bytes of LDS for " + std::to_string(m) +
                    " rows, a compute unit has " + std::to_string(CU_LDS_BYTES) + ": fewer rows a call");
    return 0;
}

// Q8_0 and EXL3 heads have the arg-max fused into the product; every other type goes through its logits (set_head keeps the
// buffer for them).
bool head_argmax_fused(const sz_session* s) { return s->head_type == SZ_TYPE_Q8_0 || head_is_exl3(s); }

// An EXL3 head (kernels/exl3.cu:349-461, 610-625 of the reference: rotate the rows once, then one pass over the matrix for all
// m <= 8 rows): the arg-max ids (0: not wanted) and / or the logits (0: not written).
int head_exl3(sz_session* s, uint32_t m, uint64_t u, uint64_t logits, uint64_t ids, uint64_t stream, const Accept* accept = nullptr) {
    const sz_session_config& c = s->cfg;
    const uint32_t kbs = c.hidden / 128, bits = (uint32_t) s->head_type - 1020;
    {
        const sz_arg a[] = {P(s->head_w), P(u), U32(c.hidden), P(s->head_xa.ptr), P(s->head_inv.ptr), U32(c.hidden)};
        if (launch("exl3_head_rotate", m, 1, 1, 64 * std::min<uint32_t>(16, kbs), 0, stream, a)) return 1;
    }
    const uint32_t nparts = c.vocab / 128, lds = exl3_head_lds_dynamic(c.hidden, m);
    const std::string kn = "head_exl3_" + std::to_string(bits);
    const sz_arg a[] = {P(s->head_w), P(s->head_xa.ptr), P(s->head_inv.ptr), P(logits), U32(c.vocab), P(s->head_part.ptr), U32(c.hidden), U32(c.vocab), U32(m), P(0)};
    if (launch(kn.c_str(), nparts, 1, 1, 256, lds, stream, a)) return 1;
    if (!ids) return 0;
    return merge_parts(s, nparts, 8, m, ids, accept, stream);
}

// The number of blocks a row may choose for a hand-off of need_k values (session.rs:5961): three quarters of k_blk, at least
// 64, when only a few are needed.
uint32_t head_proxy_k_use(const sz_session* s, uint32_t need_k) {
    const uint32_t k = s->hp.k_blk;
    return need_k <= 16 ? std::min(std::max(k * 3 / 4, 64u), k) : k;
}

// The screened head (mv_head_proxy_sparse, session.rs:5952-5995): rotate the rows, their int8 codes, the block maxima of the
// 2-bit copy, the k_use best blocks of every row, their union as a list, and the exact head on the listed blocks only.
// Leaves the list in hp.sel and the packed logits (rows max_sel * 128 apart) in hp.logits; *max_sel_out = the list's bound.
int head_proxy_sparse(sz_session* s, uint32_t m, uint64_t u, uint32_t need_k, uint32_t* max_sel_out, uint64_t stream) {
    const sz_session_config& c = s->cfg;
    const uint32_t kbs = c.hidden / 128, n_ob = c.vocab / 128, bits = (uint32_t) s->head_type - 1020;
    const uint32_t k_use = head_proxy_k_use(s, need_k), max_sel = std::min(m * k_use, n_ob);
    {
        const sz_arg a[] = {P(s->head_w), P(u), U32(c.hidden), P(s->head_xa.ptr), P(s->head_inv.ptr), U32(c.hidden)};
        if (launch("exl3_head_rotate", m, 1, 1, 64 * std::min<uint32_t>(16, kbs), 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(s->head_w), P(u), U32(c.hidden), P(s->hp.xq.ptr), P(s->hp.x_sc.ptr), P(s->hp.x_corr.ptr), U32(c.hidden)};
        if (launch("proxy_q2_quant_x", kbs, m, 1, 64, 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(s->hp.w_q2.ptr), P(s->hp.w_sc.ptr), P(s->hp.xq.ptr), P(s->hp.x_sc.ptr), P(s->hp.x_corr.ptr), P(s->hp.bmax.ptr),
                            U32(n_ob), U32(c.hidden), U32(m)};
        if (launch(m == 1 ? "proxy_q2_bmax_m1" : m <= 4 ? "proxy_q2_bmax_m4" : "proxy_q2_bmax_m8", n_ob, 1, 1, 128, 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(s->hp.bmax.ptr), U32(n_ob), U32(k_use), P(s->hp.seen.ptr)};
        if (launch("proxy_pick_rows", m, 1, 1, 1024, 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(s->hp.seen.ptr), U32(n_ob), U32(max_sel), P(s->hp.sel.ptr)};
        if (launch("proxy_compact_seen", 1, 1, 1, 64, 0, stream, a)) return 1;
    }
    const uint32_t lds = exl3_head_lds_dynamic(c.hidden, m);
    const std::string kn = "head_exl3_" + std::to_string(bits);
    const sz_arg a[] = {P(s->head_w), P(s->head_xa.ptr), P(s->head_inv.ptr), P(s->hp.logits.ptr), U32(max_sel * 128), P(s->head_part.ptr),
                        U32(c.hidden), U32(c.vocab), U32(m), P(s->hp.sel.ptr)};
    if (launch(kn.c_str(), max_sel, 1, 1, 256, lds, stream, a)) return 1;
    *max_sel_out = max_sel;
    return 0;
}

int head_logits(sz_session* s, uint32_t m, uint64_t u, uint64_t logits, uint64_t stream);

// accept (a verify round): the greedy acceptance after the ids, fused into the merge where the head has one merge for all rows
int head_argmax(sz_session* s, uint32_t m, uint64_t u, uint64_t ids, uint64_t stream, const Accept* accept = nullptr) {
    if (head_check(s, m, u, "sz_head_argmax")) return 1;
    if (!head_argmax_fused(s)) {
        // mv_cols + topk_rows_at (session.rs:7034-7052): the logits, the largest of every slice of 4096, the largest of those
        const sz_session_config& c = s->cfg;
        const uint32_t nparts = (c.vocab + 4095) / 4096;
        if (head_logits(s, m, u, s->logits.ptr, stream)) return 1;
        const sz_arg a[] = {P(s->logits.ptr), U32(c.vocab), U32(c.vocab), P(s->head_part.ptr), U32(8)};
        if (launch("argmax_slices", nparts, m, 1, 256, 0, stream, a)) return 1;
        return merge_parts(s, nparts, 8, m, ids, accept, stream);
    }
    if (head_is_exl3(s)) return head_exl3(s, m, u, 0, ids, stream, accept);
    if (head_mfma_ok(s)) return head_argmax_mfma(s, m, u, 0, ids, stream, accept);
    for (uint32_t j0 = 0; j0 < m; j0 += 4) {
        if (head_argmax_rows(s, std::min(4u, m - j0), u + (uint64_t) j0 * s->cfg.hidden * 4, 0, ids + j0 * 4ull, stream)) return 1;
    }
    if (accept) {   // the scalar head merges four rows at a time: the acceptance is a launch of its own
        const sz_arg a[] = {P(ids), P(accept->drafts), U32(m - 1), P(accept->out)};
        return launch("verify_accept", 1, 1, 1, 64, 0, stream, a);
    }
    return 0;
}

int head_logits(sz_session* s, uint32_t m, uint64_t u, uint64_t logits, uint64_t stream) {
    if (head_check(s, m, u, "sz_head_logits")) return 1;
    if (head_is_exl3(s)) return head_exl3(s, m, u, logits, 0, stream);
    if (head_mfma_ok(s)) return head_argmax_mfma(s, m, u, logits, s->ids.ptr, stream);   // one pass for all rows; the ids are a by-product
    const sz_session_config& c = s->cfg;
    return matvec_cols_dev(s->head_type, s->head_w, c.hidden, c.vocab, u, c.hidden, logits, c.vocab, m, 0, 0, stream);
}

}   // namespace

extern "C" {

sz_session* sz_session_new(const sz_session_config* cfg) {
    clear_error();
    if (ensure_init()) return nullptr;
    const sz_session_config& c = *cfg;
    if (c.hidden == 0 || c.hidden % 256 || c.ff == 0 || c.ff % 256) { fail("sz_session_new: hidden and ff must be multiples of 256"); return nullptr; }
    if (c.n_expert == 0 || c.n_expert > 512 || c.top_k == 0 || c.top_k > 16 || c.max_rows == 0 || c.max_rows > 8) {
        fail("sz_session_new: needs n_expert <= 512, top_k <= 16, max_rows <= 8");   // the planner's limits (session.rs:8190-8202)
        return nullptr;
    }
    sz_session* s = new sz_session();
    s->cfg = c;
    s->layers.resize(c.n_layers);
    if (const char* e = std::getenv("SHADOWZERO_EXPERT_MODE")) s->expert_mode = std::min(3, std::max(0, std::atoi(e)));
    const PlanLayout p = plan_layout(c.max_rows, c.top_k);
    s->GT_max = p.GT;
    const uint64_t ks_gu = exl3_ksplit(c.hidden), ks_d = exl3_ksplit(c.ff);
    const uint64_t part = std::max<uint64_t>(2ull * p.GT * ks_gu * 4 * c.ff, (uint64_t) p.GT * ks_d * 4 * c.hidden) * 4;
    const uint64_t nparts = c.vocab / 4 + 1;
    bool bad = s->plan.need(std::max(p.bytes, mma_plan(c.max_rows, c.top_k).bytes)) || s->plan2.need(std::max(p.bytes, mma_plan(c.max_rows, c.top_k).bytes)) || s->eg.need(2ull * p.R * c.ff * 4) || s->act.need((uint64_t) p.R * c.ff * 4) ||
               s->eo.need((uint64_t) p.R * c.hidden * 4) || s->part.need(part) || s->ids.need(64) ||
               s->dn.need((uint64_t) p.GT * ks_d * 4 * c.hidden * 4);
    if (c.vocab) bad = bad || s->head_part.need(nparts * 4 * 2 * 4);
    s->plan_stride = (uint32_t) ((2ull * c.max_rows * c.top_k * 4 + c.max_rows * 4 + 255) & ~255ull);
    if (c.n_layers) bad = bad || s->plans.need((uint64_t) c.n_layers * s->plan_stride);
    if (bad) {
        delete s;
        return nullptr;
    }
    return s;
}

void sz_session_free(sz_session* s) {
    if (!s) return;
    if (s->top_host) hip().hipHostFree(s->top_host);
    for (auto& g : s->graphs) sz_graph_destroy(g.second);
    delete s;
}

int32_t sz_session_set_layer_spaced(sz_session* s, uint32_t l, int32_t ty, uint64_t experts, uint64_t stride, uint64_t gap, int32_t shared_type, uint64_t shared) {
    clear_error();
    if (!s || l >= s->layers.size()) return fail("sz_session_set_layer: no layer " + std::to_string(l));
    Format f;
    std::string tag;
    if (!format_of(ty, f, tag)) return fail("sz_session_set_layer: ggml type " + std::to_string(ty) + " has no kernels");
    const sz_session_config& c = s->cfg;
    const uint64_t gu = matrix_bytes(f, c.hidden, c.ff) + gap, dn = matrix_bytes(f, c.ff, c.hidden);   // gu: from a projection to the next
    if (stride < 2 * gu + dn) return fail("sz_session_set_layer: the expert stride is smaller than an expert");
    if ((experts | stride | shared | gap) & 3) return fail("sz_session_set_layer: expert blobs must be 4-byte aligned");
    if (gu >> 32) return fail("sz_session_set_layer: a projection of 4 GiB or more");
    SzLayer& L = s->layers[l];
    // the address table eaddr[part * ne + e] (session.rs:2129-2146), then the shared expert's three parts
    std::vector<uint64_t> tab(3ull * c.n_expert + 3);
    for (uint32_t e = 0; e < c.n_expert; e++) {
        const uint64_t b = experts + e * stride;
        tab[e] = b;
        tab[c.n_expert + e] = b + gu;
        tab[2ull * c.n_expert + e] = b + 2 * gu;
    }
    Format fs;
    std::string tags;
    if (shared) {
        if (!format_of(shared_type, fs, tags)) return fail("sz_session_set_layer: shared type " + std::to_string(shared_type) + " has no kernels");
        const uint64_t sgu = matrix_bytes(fs, c.hidden, c.ff) + gap;
        tab[3ull * c.n_expert] = shared;
        tab[3ull * c.n_expert + 1] = shared + sgu;
        tab[3ull * c.n_expert + 2] = shared + 2 * sgu;
    }
    if (L.eaddr.need(tab.size() * 8) || sz_upload(L.eaddr.ptr, tab.data(), tab.size() * 8)) return 1;
    L.type = ty;
    L.shared_type = shared_type;
    L.experts = experts;
    L.stride = stride;
    L.shared = shared;
    L.gap = gap;
    L.set = true;
    for (auto& g : s->graphs) sz_graph_destroy(g.second);   // captured address tables may be stale
    s->graphs.clear();
    return 0;
}

int32_t sz_session_set_layer(sz_session* s, uint32_t l, int32_t ty, uint64_t experts, uint64_t stride, int32_t shared_type, uint64_t shared) {
    return sz_session_set_layer_spaced(s, l, ty, experts, stride, 0, shared_type, shared);
}

// Where a layer's experts should lie for their rows to start on 128-byte lines of memory.  An EXL3 projection's trellis
// begins 2 (in + out) + 4 bytes into its blob (exl3.rs:390-393), and a launch fetches a row of it in segments of 512 to
// 2048 bytes: 4 bytes off a line, every segment touches one line more than it fills.  With the first blob `lead` bytes past
// a 128-byte boundary, `gap` bytes between an expert's projections and a stride that is a multiple of 128, every trellis
// starts on a line.  GGUF rows (34- and 110-byte blocks) have no such boundary: lead and gap 0.
void sz_layer_spacing(int32_t ty, uint64_t hidden, uint64_t ff, uint32_t* lead, uint32_t* gap) {
    Format f;
    std::string tag;
    uint32_t ld = 0, gp = 0;
    if (format_of(ty, f, tag) && f.exl3) {
        ld = (uint32_t) ((128 - (2 * (hidden + ff) + 4) % 128) % 128);
        gp = (uint32_t) ((128 - matrix_bytes(f, hidden, ff) % 128) % 128);
    }
    if (lead) *lead = ld;
    if (gap) *gap = gp;
}

int32_t sz_session_set_router(sz_session* s, uint32_t l, int32_t rty, uint64_t rw, int32_t gty, uint64_t gw) {
    clear_error();
    if (!s || l >= s->layers.size()) return fail("sz_session_set_router: no layer " + std::to_string(l));
    const sz_session_config& c = s->cfg;
    Format fr, fg;
    std::string tr, tg;
    if (!format_of(rty, fr, tr) || !fr.dense) return fail("sz_session_set_router: the router must be F32, F16 or BF16");
    if (gw && (!format_of(gty, fg, tg) || !fg.dense)) return fail("sz_session_set_router: the shared expert's gate must be F32, F16 or BF16");
    if (!rw || (rw & (4 * fr.bb - 1)) || (gw & (4 * (gw ? fg.bb : 1) - 1))) return fail("sz_session_set_router: matrices must be aligned to four weights");
    if (s->rl.need((uint64_t) c.max_rows * c.n_expert * 4) || s->sgl.need((uint64_t) c.max_rows * 4)) return 1;
    auto code = [](int ty) { return ty == SZ_TYPE_F32 ? 0u : ty == SZ_TYPE_F16 ? 1u : 2u; };
    DenseJob jobs[2];
    const uint32_t g0 = dense_groups(c.n_expert, c.hidden);
    jobs[0] = {rw, s->rl.ptr, c.n_expert, c.n_expert, code(rty), 0, 0, 1.0f};
    jobs[1] = {gw, s->sgl.ptr, 1, gw ? 1u : 0u, code(gty), g0, 0, 1.0f};
    SzLayer& L = s->layers[l];
    if (L.jobs.need(sizeof jobs) || sz_upload(L.jobs.ptr, jobs, sizeof jobs)) return 1;
    L.router_groups = g0 + (gw ? dense_groups(1, c.hidden) : 0);
    for (auto& g : s->graphs) sz_graph_destroy(g.second);
    s->graphs.clear();
    return 0;
}

int32_t sz_moe_router_verify(sz_session* s, uint32_t l, uint32_t m, uint64_t u, uint64_t stream) {
    clear_error();
    if (!s || l >= s->layers.size() || !s->layers[l].router_groups) return fail("sz_moe_router_verify: layer " + std::to_string(l) + " has no router set");
    const sz_session_config& c = s->cfg;
    if (m == 0 || m > c.max_rows) return fail("sz_moe_router_verify: " + std::to_string(m) + " rows (1.." + std::to_string(c.max_rows) + ")");
    if (u & 15) return fail("sz_moe_router_verify: activations must be 16-byte aligned");
    const SzLayer& L = s->layers[l];
    const sz_arg a[] = {P(L.jobs.ptr), U32(2), P(u), U32(c.hidden), U32(c.hidden), U32(m)};
    return launch("matvec_cols_multi", L.router_groups, 1, 1, 256, dense_lds(c.hidden, m), stream, a);
}

int32_t sz_session_router_outputs(sz_session* s, uint64_t* rl, uint64_t* sgl) {
    clear_error();
    if (!s || !s->rl.ptr) return fail("sz_session_router_outputs: no router set");
    *rl = s->rl.ptr;
    *sgl = s->sgl.ptr;
    return 0;
}

int32_t sz_moe_block_verify(sz_session* s, uint32_t l, uint32_t m, uint64_t u, uint64_t y, uint64_t stream) {
    if (sz_moe_router_verify(s, l, m, u, stream)) return 1;
    return moe_layer(s, l, m, u, s->rl.ptr, s->sgl.ptr, y, stream);
}

int32_t sz_session_set_head(sz_session* s, int32_t ty, uint64_t w) {
    clear_error();
    if (!s) return fail("sz_session_set_head: null session");
    const bool exl3 = ty >= 1021 && ty <= 1028;
    const bool plain = ty == SZ_TYPE_F32 || ty == SZ_TYPE_F16 || ty == SZ_TYPE_BF16;
    if (ty != SZ_TYPE_Q8_0 && ty != SZ_TYPE_IQ3_S && !plain && !exl3)
        return fail("sz_session_set_head: the head must be Q8_0, IQ3_S, F32, F16, BF16 or EXL3 at a whole bit rate");
    // a type without a fused arg-max keeps its logits: allocated here, never during a call (a call may be under capture)
    if (ty != SZ_TYPE_Q8_0 && !exl3 && s->logits.need((uint64_t) s->cfg.max_rows * s->cfg.vocab * 4)) return 1;
    if (w & 15) return fail("sz_session_set_head: the head must be 16-byte aligned");
    if (exl3) {
        const sz_session_config& c = s->cfg;
        if (c.vocab == 0 || c.vocab % 128 || c.hidden % 128 || c.hidden > 8192) return fail("sz_session_set_head: an EXL3 head needs hidden (<= 8192) and the vocabulary to be multiples of 128");
        // a head that cannot take even one row is refused here; how many rows a call may bring is checked call by call
        if (exl3_head_lds((uint32_t) ty - 1020, c.hidden, 1) > CU_LDS_BYTES)
            return fail("sz_session_set_head: an EXL3 head of hidden " + std::to_string(c.hidden) + " does not fit a compute unit's LDS");
        if (s->head_xa.need((uint64_t) c.hidden / 128 * 16 * 256) || s->head_inv.need(64)) return 1;
    }
    s->head_type = ty;
    s->head_w = w;
    s->hp.k_blk = 0;   // a screen belongs to the head it was built from
    for (auto& g : s->graphs) sz_graph_destroy(g.second);
    s->graphs.clear();
    return 0;
}

uint32_t sz_exl3_head_lds_bytes(int32_t ty, uint32_t hidden, uint32_t m) {
    return (ty >= 1021 && ty <= 1028) ? exl3_head_lds((uint32_t) ty - 1020, hidden, m) : 0;
}

int32_t sz_session_set_head_proxy(sz_session* s, uint32_t k_blk) {
    clear_error();
    if (!s) return fail("sz_session_set_head_proxy: null session");
    if (k_blk == 0) {
        s->hp.k_blk = 0;
        return 0;
    }
    const sz_session_config& c = s->cfg;
    if (!head_is_exl3(s)) return fail("sz_session_set_head_proxy: the screen is built from an EXL3 head (set one first)");
    if (c.hidden > 4096) return fail("sz_session_set_head_proxy: hidden above 4096");      // session.rs:2656
    const uint64_t n_ob = c.vocab / 128, n_b = c.hidden / 128, rows = 8;
    const uint32_t k = (uint32_t) std::min<uint64_t>(std::max<uint32_t>(k_blk, 16), n_ob);   // session.rs:2659
    const uint64_t max_sel = std::min<uint64_t>(rows * k, n_ob);
    if ((max_sel * 128 + 4095) / 4096 > 64) return fail("sz_session_set_head_proxy: 8 rows of k_blk blocks are more than the top-64 merge takes (k_blk <= 256)");
    auto& h = s->hp;
    if (h.w_q2.need((uint64_t) c.vocab * c.hidden / 4) || h.w_sc.need((uint64_t) c.vocab * n_b * 2) || h.xq.need(rows * n_b * 32 * 4) ||
        h.x_sc.need(rows * n_b * 4) || h.x_corr.need(rows * n_b * 4) || h.bmax.need(rows * n_ob * 4) || h.seen.need((n_ob + 31) / 32 * 4) ||
        h.sel.need((1 + max_sel) * 4) || h.logits.need(rows * max_sel * 128 * 4))
        return 1;
    if (sz_memset(h.seen.ptr, 0, h.seen.bytes, 0) || sz_memset(h.xq.ptr, 0, h.xq.bytes, 0) || sz_memset(h.x_sc.ptr, 0, h.x_sc.bytes, 0) ||
        sz_memset(h.x_corr.ptr, 0, h.x_corr.bytes, 0))
        return 1;
    const std::string kn = "exl3_build_q2_proxy_" + std::to_string(s->head_type - 1020);
    const sz_arg a[] = {P(s->head_w), P(h.w_q2.ptr), P(h.w_sc.ptr), U32(c.hidden), U32(c.vocab)};
    if (launch(kn.c_str(), (uint32_t) n_ob, (uint32_t) n_b, 1, 256, 0, 0, a)) return 1;
    if (sz_stream_synchronize(0)) return 1;
    h.k_blk = k;
    return 0;
}

uint64_t sz_session_buffer(sz_session* s, int32_t which) {
    if (!s) return 0;
    const uint64_t at[] = {s->last_plan ? s->last_plan : s->plan.ptr, s->part.ptr, s->dn.ptr, s->eg.ptr, s->eo.ptr, s->hp.w_q2.ptr, s->hp.w_sc.ptr, s->hp.xq.ptr, s->hp.x_sc.ptr,
                           s->hp.x_corr.ptr, s->hp.bmax.ptr, s->hp.sel.ptr, s->hp.logits.ptr, s->pf.gup.ptr, s->pf.eo.ptr, s->pf.arows.ptr, s->pf.ainv.ptr, s->pf.items.ptr};
    return which >= 0 && which < (int32_t) (sizeof at / sizeof at[0]) ? at[which] : 0;
}

int32_t sz_session_set_expert_mode(sz_session* s, int32_t mode) {
    clear_error();
    if (!s) return fail("sz_session_set_expert_mode: null session");
    if (mode < 0 || mode > 3)
        return fail("sz_session_set_expert_mode: mode " + std::to_string(mode) + " (0 exact, 1 matrix cores, 2 matrix cores with the linearised codebook, 3 exact decode with f16 inputs)");
    if (s->expert_mode != mode) {
        for (auto& g : s->graphs) sz_graph_destroy(g.second);   // a captured round holds the other mode's launches
        s->graphs.clear();
    }
    s->expert_mode = mode;
    return 0;
}

int32_t sz_session_set_graph(sz_session* s, int32_t enabled) {
    clear_error();
    if (!s) return fail("sz_session_set_graph: null session");
    s->use_graph = enabled != 0;
    return 0;
}

int32_t sz_moe_layer_verify(sz_session* s, uint32_t l, uint32_t m, uint64_t u, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_moe_layer_verify: null session");
    return moe_layer(s, l, m, u, rl, sgl, y, stream);
}

int32_t sz_session_last_route(sz_session* s, uint32_t m, uint32_t* idx, float* w, uint64_t stream) {
    clear_error();
    if (!s || m == 0 || m > s->cfg.max_rows) return fail("sz_session_last_route: bad arguments");
    if (sz_stream_synchronize(stream)) return 1;
    const PlanLayout p = plan_layout(m, s->cfg.top_k);
    const uint64_t n = (uint64_t) m * s->cfg.top_k * 4;
    const uint64_t plan = s->last_plan ? s->last_plan : s->plan.ptr;
    if (s->last_fused) return sz_download(idx, plan, n) || sz_download(w, plan + n, n);
    if (sz_download(idx, plan + p.tidx_off, n)) return 1;
    return sz_download(w, plan + p.w_off, n);
}

int32_t sz_head_argmax(sz_session* s, uint32_t m, uint64_t u, uint64_t ids, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_head_argmax: null session");
    return head_argmax(s, m, u, ids, stream);
}

int32_t sz_head_logits(sz_session* s, uint32_t m, uint64_t u, uint64_t logits, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_head_logits: null session");
    return head_logits(s, m, u, logits, stream);
}

// The merge kernel's output goes straight into pinned host memory (device-visible, coherent): once the stream has drained the
// 2 KiB a row are there, and no copy from device memory (a blocking driver call of its own) is needed.
static int top_finish(sz_session* s, uint32_t m, uint32_t* top_host, uint64_t stream) {
    if (sz_stream_synchronize(stream)) return 1;
    std::memcpy(top_host, s->top_host, (size_t) m * 128 * 4);
    return 0;
}

int32_t sz_head_top(sz_session* s, uint32_t m, uint64_t u, uint32_t* top_host, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_head_top: null session");
    if (!s->top_host && hip_check(hip().hipHostMalloc(&s->top_host, 8 * 128 * 4, 0), "hipHostMalloc")) return 1;
    const uint64_t topo = (uint64_t) s->top_host;
    const sz_session_config& c = s->cfg;
    const uint32_t nb = (c.vocab + 4095) / 4096;
    if (nb > 64) return fail("sz_head_top: vocabulary above 262144");
    if (head_check(s, m, u, "sz_head_top")) return 1;
    if (s->hp.k_blk) {   // head_top_at, session.rs:5997-6022: the screened form, the top 64 among the chosen blocks
        if (s->topv.need(8ull * 64 * 64 * 4) || s->topi.need(8ull * 64 * 64 * 4)) return 1;
        uint32_t max_sel = 0;
        if (head_proxy_sparse(s, m, u, 64, &max_sel, stream)) return 1;
        const uint32_t nbs = (max_sel * 128 + 4095) / 4096;
        const sz_arg a[] = {P(s->hp.logits.ptr), U32(max_sel * 128), P(s->hp.sel.ptr), U32(nbs), P(s->topv.ptr), P(s->topi.ptr)};
        if (launch("topk_slices_blks", m * nbs, 1, 1, 1024, 0, stream, a)) return 1;
        const sz_arg b[] = {P(s->topv.ptr), P(s->topi.ptr), U32(nbs), P(topo)};
        if (launch("topk_merge", m, 1, 1, 1024, 0, stream, b)) return 1;
        return top_finish(s, m, top_host, stream);
    }
    if (s->logits.need((uint64_t) c.max_rows * c.vocab * 4) || s->topv.need((uint64_t) c.max_rows * nb * 64 * 4) ||
        s->topi.need((uint64_t) c.max_rows * nb * 64 * 4))
        return 1;
    if (head_logits(s, m, u, s->logits.ptr, stream)) return 1;
    const sz_arg a[] = {P(s->logits.ptr), U32(c.vocab), U32(c.vocab), U32(nb), P(s->topv.ptr), P(s->topi.ptr)};
    if (launch("topk_slices", m * nb, 1, 1, 1024, 0, stream, a)) return 1;
    const sz_arg b[] = {P(s->topv.ptr), P(s->topi.ptr), U32(nb), P(topo)};
    if (launch("topk_merge", m, 1, 1, 1024, 0, stream, b)) return 1;
    return top_finish(s, m, top_host, stream);
}

int32_t sz_verify_accept(const uint32_t* ids, const uint32_t* drafts, uint32_t n_drafts, uint32_t* keep) {
    clear_error();
    uint32_t k = 1;
    for (uint32_t i = 0; i < n_drafts; i++) {
        if (ids[i] != drafts[i]) break;
        k++;
    }
    *keep = k;
    return 0;
}

int32_t sz_lookup_draft(const uint32_t* hist, uint64_t n_hist, uint32_t k, const uint32_t* lens, uint32_t n_lens, uint32_t* drafts, uint32_t* n_drafts) {
    clear_error();
    if (!n_drafts || (n_hist && !hist) || (n_lens && !lens) || (k && !drafts)) return fail("sz_lookup_draft: null argument");
    *n_drafts = 0;
    for (uint32_t li = 0; li < n_lens; li++) {
        const uint64_t n = lens[li];
        if (k == 0 || n_hist <= n) break;   // as the reference: a length the history cannot hold ends the search
        const uint32_t* tail = hist + n_hist - n;
        for (uint64_t i = n_hist - n; i-- > 0;) {   // the most recent earlier occurrence first
            if (std::memcmp(hist + i, tail, n * 4) != 0) continue;
            const uint64_t end = std::min<uint64_t>(i + n + k, n_hist);
            for (uint64_t j = i + n; j < end; j++) drafts[(*n_drafts)++] = hist[j];
            return 0;
        }
    }
    return 0;
}

int32_t sz_verify_round(sz_session* s, uint32_t m, uint64_t u, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t head_u, uint64_t drafts,
                        uint64_t out, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_verify_round: null session");
    if (m == 0 || m > s->cfg.max_rows) return fail("sz_verify_round: " + std::to_string(m) + " rows");
    const sz_session_config& c = s->cfg;
    // everything that can be refused is refused before a capture begins
    if (head_check(s, m, head_u, "sz_verify_round")) return 1;
    for (uint32_t l = 0; l < c.n_layers; l++)
        if (!s->layers[l].set) return fail("sz_verify_round: layer " + std::to_string(l) + " has no experts set");
    const SzGraphKey key{{m, u, rl, sgl, y, head_u, drafts, out, stream, 0}};
    auto it = s->use_graph ? s->graphs.find(key) : s->graphs.end();
    if (it == s->graphs.end()) {
        static const bool no_graph = std::getenv("SHADOWZERO_NO_GRAPH") != nullptr;
        auto record = [&]() -> int {
            // an EXL3 layer's rank-order sum rides the first launch of the layer after it; the last layer's gets its own launch
            PendingSum ps;
            bool any_exl3 = false;
            for (uint32_t l = 0; l < c.n_layers; l++) any_exl3 = any_exl3 || (s->layers[l].type >= 1021 && s->layers[l].type <= 1033);
            static const bool route_in_launch = std::getenv("SHADOWZERO_ROUTE_IN_LAUNCH") != nullptr;   // the form without the routing launch, for comparisons
            if (any_exl3 && (s->expert_mode == 0 || s->expert_mode == 3) && !route_in_launch && c.n_layers >= 12) {
                // every layer's router logits are inputs of the round: all of them are routed by one launch before the first layer
                // (about 10 us, against about 1 us a layer that the selection inside launch 1 costs: not for short rounds)
                const sz_arg a[] = {P(rl), P(s->plans.ptr), U32(s->plan_stride), U32(c.n_expert), U32(c.top_k), U32(m), U32(c.n_layers)};
                if (launch("verify_route_layers", (c.n_layers * m + 3) / 4, 1, 1, 256, 0, stream, a)) return 1;
                ps.plans = s->plans.ptr;
                ps.plan_stride = s->plan_stride;
            }
            for (uint32_t l = 0; l < c.n_layers; l++) {
                const uint64_t off = (uint64_t) l * m;
                if (moe_layer(s, l, m, u + off * c.hidden * 4, rl + off * c.n_expert * 4, sgl + off * 4, y + off * c.hidden * 4, stream, &ps)) return 1;
            }
            if (launch_pending_sum(s, ps, m, stream)) return 1;
            const Accept acc{drafts, out};
            return head_argmax(s, m, head_u, out + 8, stream, &acc);
        };
        if (no_graph || !s->use_graph || stream == 0) return record();   // the null stream cannot be captured
        if (sz_capture_begin(stream)) return 1;
        const int r = record();
        const std::string err = r ? sz_last_error() : "";
        uint64_t exec = 0;
        const int e = sz_capture_end(stream, &exec);
        if (r) {
            if (!e && exec) sz_graph_destroy(exec);   // a graph of a round that could not be recorded is not kept
            return fail(err);
        }
        if (e) return 1;
        it = s->graphs.emplace(key, exec).first;
    }
    return sz_graph_launch(it->second, stream);
}

int32_t sz_quantize_act(uint64_t x, uint64_t n, uint64_t q, uint64_t d, uint64_t stream) {
    clear_error();
    if (n % 32) return fail("sz_quantize_act: the length must be a multiple of 32");
    if (n == 0) return 0;
    const sz_arg a[] = {P(x), U64(n), P(q), P(d)};
    return launch("quant_act_q8", (uint32_t) ((n / 32 + 255) / 256), 1, 1, 256, 0, stream, a);
}

int32_t sz_moe_prefill_chunk(sz_session* s, uint32_t l, uint32_t tokens, uint64_t x, uint64_t rl, uint64_t sgl, uint64_t y, uint64_t stream) {
    clear_error();
    if (!s) return fail("sz_moe_prefill_chunk: null session");
    const sz_session_config& c = s->cfg;
    if (l >= s->layers.size() || !s->layers[l].set) return fail("sz_moe_prefill_chunk: layer " + std::to_string(l) + " has no experts set");
    SzLayer& L = s->layers[l];
    Format f;
    std::string tag;
    format_of(L.type, f, tag);
    const bool exl3 = f.exl3 && !f.half;
    if ((L.type != SZ_TYPE_IQ3_S && !exl3) || (L.shared && L.shared_type != L.type))
        return fail("sz_moe_prefill_chunk: the chunk kernels are built for IQ3_S experts (int8 activations) and EXL3 experts at a whole bit rate");
    if (tokens == 0 || tokens > 16384) return fail("sz_moe_prefill_chunk: " + std::to_string(tokens) + " tokens (1..16384)");   // BIG_BATCH_MAX, session.rs:191
    if (c.hidden % 256 || c.ff % 256 || (x & 15) || (y & 15)) return fail("sz_moe_prefill_chunk: shapes must be multiples of 256 and 16-byte aligned");
    const bool shared = L.shared != 0;
    const uint64_t T = tokens, k = c.top_k, np = T * k, rows = np + (shared ? T : 0);
    auto& pb = s->pf;
    if (exl3) {
        // EXL3 experts: f16 activations on the columns of the matrix instruction, the rotations on the matrix cores too, items of
        // up to `tok` pairs (kernels/exl3.hip, "the prefill chunk of an EXL3 layer": XPF_NT, XPF_TOK, XPF_LDS_WORDS)
        if (c.ff > 512) return fail("sz_moe_prefill_chunk: EXL3 experts of more than 512 intermediate features are not built (a workgroup keeps four 128-blocks of a token)");
        const uint32_t zs = (c.hidden / 128 + 3) / 4;
        const uint32_t tok = 16 * (f.bits <= 7 ? 3 : 2), depth = f.bits <= 2 ? 8 : f.bits <= 5 ? 6 : 4;   // XPF_NT, XPF_D
        const uint64_t max_items = c.n_expert + 1 + rows / tok;
        if (pb.tidx.need(np * 4) || pb.w.need(np * 4) || pb.cnt.need(T * 4) || pb.offs.need((c.n_expert + 2) * 4ull) || pb.list.need(rows * 4) ||
            pb.items.need((2 + 4 * max_items) * 4) || pb.gup.need(2ull * rows * zs * c.ff * 4) || pb.eo.need(rows * c.hidden * 4) ||
            pb.arows.need(max_items * tok * 1024) || pb.ainv.need(max_items * tok * 4))
            return 1;
        const uint64_t sh = shared ? L.eaddr.ptr + 3ull * c.n_expert * 8 : 0, items_d = pb.items.ptr + (1 + 2 * max_items) * 4;
        {
            const sz_arg a[] = {P(rl), P(pb.tidx.ptr), P(pb.w.ptr), U32(c.n_expert), U32(c.top_k), U32(tokens)};
            if (launch("route_topk_rows", (tokens + 3) / 4, 1, 1, 256, 0, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(pb.tidx.ptr), U32(tokens), U32(c.top_k), U32(c.n_expert), U32(shared ? tokens : 0), P(pb.offs.ptr), P(pb.list.ptr), P(pb.cnt.ptr),
                                P(pb.items.ptr), P(items_d), U32(tok), U32(tok)};
            if (launch("prefill_group", 1, 1, 1, 1024, 0, stream, a)) return 1;
        }
        const uint32_t stride = (f.bits == 3 || f.bits == 4) ? 4 : (uint32_t) f.bits;
        const uint32_t lds = 4 * (tok / 16 * 4096 + 4 * (depth * 64 * stride) + 2 * tok + 4 * tok + tok);   // XPF_LDS_WORDS
        {
            const sz_arg a[] = {P(L.eaddr.ptr), P(sh), P(pb.offs.ptr), P(pb.list.ptr), P(pb.items.ptr), P(x), P(pb.gup.ptr), U32(c.n_expert), U32(c.top_k),
                                U32((uint32_t) np), U32((uint32_t) rows), U32(c.hidden), U32(c.ff)};
            if (launch(("prefill_gate_up_" + tag).c_str(), (uint32_t) max_items, 2 * zs, 1, 256, lds, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(L.eaddr.ptr), P(sh), P(pb.offs.ptr), P(pb.list.ptr), P(pb.items.ptr), P(pb.gup.ptr), P(pb.arows.ptr), P(pb.ainv.ptr), U32(c.n_expert),
                                U32(c.top_k), U32((uint32_t) np), U32((uint32_t) rows), U32(c.hidden), U32(c.ff), U32(zs), U32(tok)};
            if (launch("prefill_act_exl3", (uint32_t) max_items, tok / 16, 1, 256, 0, stream, a)) return 1;
        }
        {
            const sz_arg a[] = {P(L.eaddr.ptr), P(sh), P(pb.offs.ptr), P(pb.list.ptr), P(pb.items.ptr), P(pb.arows.ptr), P(pb.ainv.ptr), P(pb.eo.ptr), U32(c.n_expert),
                                U32(c.top_k), U32((uint32_t) np), U32(c.hidden), U32(c.ff)};
            if (launch(("prefill_down_" + tag).c_str(), (uint32_t) max_items, (c.hidden / 128 + 3) / 4, 1, 256, lds, stream, a)) return 1;
        }
        const sz_arg a[] = {P(y), P(pb.eo.ptr), P(pb.w.ptr), P(shared ? pb.eo.ptr + np * c.hidden * 4 : 0), P(sgl), P(pb.cnt.ptr), U32(c.hidden), U32(c.top_k)};
        return launch("moe_combine_qwen_rows", (c.hidden + 255) / 256, tokens, 1, 256, 0, stream, a);
    }
    const uint64_t max_items = c.n_expert + 1 + rows / 64, max_items_d = c.n_expert + 1 + rows / 32;   // every expert's runs of up to 64 (32) pairs: PF_TOK, PF_TOK_D in kernels/prefill.hip
    if (pb.xq.need(T * c.hidden) || pb.xd.need(T * c.hidden / 32 * 4) || pb.tidx.need(np * 4) || pb.w.need(np * 4) || pb.cnt.need(T * 4) ||
        pb.offs.need((c.n_expert + 2) * 4ull) || pb.list.need(rows * 4) || pb.items.need((2 + 2 * max_items + 2 * max_items_d) * 4) || pb.hq.need(rows * c.ff) || pb.hd.need(rows * (c.ff / 32) * 4) ||
        pb.eo.need(rows * c.hidden * 4))
        return 1;
    const uint64_t sh = shared ? L.eaddr.ptr + 3ull * c.n_expert * 8 : 0;
    {
        // routing and quantization do not depend on each other: one launch
        const uint64_t n = T * c.hidden;
        const sz_arg a[] = {P(x), U64(n), P(pb.xq.ptr), P(pb.xd.ptr), P(rl), P(pb.tidx.ptr), P(pb.w.ptr), U32(c.n_expert), U32(c.top_k), U32(tokens)};
        if (launch("prefill_front", (tokens + 3) / 4 + (uint32_t) ((n / 32 + 255) / 256), 1, 1, 256, 0, stream, a)) return 1;
    }
    const uint64_t items_d = pb.items.ptr + (1 + 2 * max_items) * 4;   // the down kernel's items: runs of up to 32 pairs (PF_TOK_D)
    {
        const sz_arg a[] = {P(pb.tidx.ptr), U32(tokens), U32(c.top_k), U32(c.n_expert), U32(shared ? tokens : 0), P(pb.offs.ptr), P(pb.list.ptr), P(pb.cnt.ptr), P(pb.items.ptr), P(items_d), U32(64), U32(32)};
        if (launch("prefill_group", 1, 1, 1, 1024, 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(L.eaddr.ptr), P(sh), P(pb.offs.ptr), P(pb.list.ptr), P(pb.items.ptr), P(pb.xq.ptr), P(pb.xd.ptr), P(pb.hq.ptr), P(pb.hd.ptr),
                            U32(c.n_expert), U32(c.top_k), U32((uint32_t) np), U32(c.hidden), U32(c.ff)};
        static const bool w4 = std::getenv("SHADOWZERO_PREFILL_FOUR_WAVES") != nullptr;   // the four-wave form, for comparisons
        if (launch(w4 ? "prefill_gate_up_iq3_s_w4" : "prefill_gate_up_iq3_s", c.ff / 64, (uint32_t) max_items, 1, w4 ? 256 : 512, 0, stream, a)) return 1;
    }
    {
        // a workgroup takes 4 (else 2, else 1) blocks of 64 rows in turn: the two chunks of one block are too little work for its set-up
        const uint32_t blocks = c.hidden / 64, per = blocks % 4 == 0 ? 4 : blocks % 2 == 0 ? 2 : 1;
        const sz_arg a[] = {P(L.eaddr.ptr), P(sh), P(pb.offs.ptr), P(pb.list.ptr), P(items_d), P(pb.hq.ptr), P(pb.hd.ptr), P(pb.eo.ptr), U32(c.n_expert),
                            U32(c.hidden), U32(c.ff)};
        if (launch("prefill_down_iq3_s", blocks / per, (uint32_t) max_items_d, 1, 256, 0, stream, a)) return 1;
    }
    const sz_arg a[] = {P(y), P(pb.eo.ptr), P(pb.w.ptr), P(shared ? pb.eo.ptr + np * c.hidden * 4 : 0), P(sgl), P(pb.cnt.ptr), U32(c.hidden), U32(c.top_k)};
    return launch("moe_combine_qwen_rows", (c.hidden + 255) / 256, tokens, 1, 256, 0, stream, a);
}

// The chunk's intermediate buffers, for tests: which = 0 xq (int8), 1 xd (f32), 2 tidx (u32), 3 w (f32), 4 hq (int8), 5 hd (f32),
// 6 eo (f32).  Returns the device address (0 if the session has not run a chunk).
uint64_t sz_prefill_buffer(sz_session* s, int32_t which) {
    if (!s) return 0;
    auto& pb = s->pf;
    const uint64_t ptrs[] = {pb.xq.ptr, pb.xd.ptr, pb.tidx.ptr, pb.w.ptr, pb.hq.ptr, pb.hd.ptr, pb.eo.ptr};
    return which >= 0 && which < 7 ? ptrs[which] : 0;
}

}   // extern "C"

// ---- the hyper-connection around a sublayer ---------------------------------------------------------------------------------
struct sz_hc {
    sz_hc_config cfg{};
    DevBuf rn, down, mix, g, jobs;   // [max_rows][ch], [max_rows][rank], [max_rows][ch], [max_rows][streams], 3 jobs
    uint32_t groups_di = 0, groups_up = 0;
};

extern "C" {

sz_hc* sz_hc_new(const sz_hc_config* cfg) {
    clear_error();
    if (ensure_init()) return nullptr;
    const sz_hc_config& c = *cfg;
    const uint64_t ch = (uint64_t) c.hidden * c.streams;
    Format fd, fu, fi;
    std::string td, tu, ti;
    if (c.hidden == 0 || c.hidden % 4 || c.streams == 0 || c.streams > 64 || c.rank == 0 || c.rank % 4 || c.max_rows == 0 || c.max_rows > 8 || ch >> 31) {
        fail("sz_hc_new: hidden and rank must be multiples of 4, streams 1..64, max_rows 1..8");
        return nullptr;
    }
    if (!format_of(c.down_type, fd, td) || !fd.dense || !format_of(c.up_type, fu, tu) || !fu.dense ||
        (c.inject_w && (!format_of(c.inject_type, fi, ti) || !fi.dense))) {
        fail("sz_hc_new: the projections must be F32, F16 or BF16");
        return nullptr;
    }
    if (!c.norm_w || !c.down_w || !c.up_w || (c.norm_w & 3) || (c.down_w & (4 * fd.bb - 1)) || (c.up_w & (4 * fu.bb - 1)) ||
        (c.inject_w & (4 * (c.inject_w ? fi.bb : 1) - 1))) {
        fail("sz_hc_new: weights must be resident and aligned to four weights");
        return nullptr;
    }
    sz_hc* h = new sz_hc();
    h->cfg = c;
    if (h->rn.need(c.max_rows * ch * 4) || h->down.need((uint64_t) c.max_rows * c.rank * 4) || h->mix.need(c.max_rows * ch * 4) ||
        h->g.need((uint64_t) c.max_rows * c.streams * 4) || h->jobs.need(3 * sizeof(DenseJob))) {
        delete h;
        return nullptr;
    }
    auto code = [](int ty) { return ty == SZ_TYPE_F32 ? 0u : ty == SZ_TYPE_F16 ? 1u : 2u; };
    const uint32_t gd = dense_groups(c.rank, ch);
    DenseJob jobs[3];
    jobs[0] = {c.down_w, h->down.ptr, c.rank, c.rank, code(c.down_type), 0, 1, (float) c.streams};                    // silu(v / cs)
    jobs[1] = {c.inject_w, h->g.ptr, c.streams, c.inject_w ? c.streams : 0u, code(c.inject_type), gd, 2, (float) c.streams};   // 2 sigmoid(v / cs)
    jobs[2] = {c.up_w, h->mix.ptr, (uint32_t) ch, (uint32_t) ch, code(c.up_type), 0, 3, 1.0f};                         // sigmoid(v)
    h->groups_di = gd + (c.inject_w ? dense_groups(c.streams, ch) : 0);
    h->groups_up = dense_groups(ch, c.rank);
    if (sz_upload(h->jobs.ptr, jobs, sizeof jobs)) {
        delete h;
        return nullptr;
    }
    return h;
}

void sz_hc_free(sz_hc* h) { delete h; }
uint64_t sz_hc_gains(sz_hc* h) { return h ? h->g.ptr : 0; }

int32_t sz_hc_read(sz_hc* h, uint32_t m, uint64_t r, uint64_t u, uint64_t stream) {
    clear_error();
    if (!h) return fail("sz_hc_read: null handle");
    const sz_hc_config& c = h->cfg;
    if (m == 0 || m > c.max_rows) return fail("sz_hc_read: " + std::to_string(m) + " rows (1.." + std::to_string(c.max_rows) + ")");
    if ((r & 15) || (u & 15)) return fail("sz_hc_read: rows must be 16-byte aligned");
    const uint32_t ch = c.hidden * c.streams;
    {
        const sz_arg a[] = {P(r), P(c.norm_w), P(h->rn.ptr), U32(c.hidden), F32(c.eps), U32(c.streams)};
        if (launch("rmsnorm_groups_rows", c.streams, m, 1, 256, 0, stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(h->jobs.ptr), U32(2), P(h->rn.ptr), U32(ch), U32(ch), U32(m)};
        if (launch("matvec_cols_multi", h->groups_di, 1, 1, 256, dense_lds(ch, m), stream, a)) return 1;
    }
    {
        const sz_arg a[] = {P(h->jobs.ptr + 2 * sizeof(DenseJob)), U32(1), P(h->down.ptr), U32(c.rank), U32(c.rank), U32(m)};
        if (launch("matvec_cols_multi", h->groups_up, 1, 1, 256, dense_lds(c.rank, m), stream, a)) return 1;
    }
    const sz_arg a[] = {P(h->rn.ptr), P(h->mix.ptr), P(u), U32(c.hidden), U32(c.streams)};
    return launch("hc_mix_rows", (c.hidden + 255) / 256, m, 1, 256, 0, stream, a);
}

int32_t sz_hc_write(uint64_t r, uint64_t g, uint64_t y, uint32_t m, uint32_t hidden, uint32_t streams, uint64_t stream) {
    clear_error();
    if (m == 0 || hidden == 0 || streams == 0 || streams > 65535 || m > 65535) return fail("sz_hc_write: bad shape");
    const sz_arg a[] = {P(r), P(g), P(y), U32(hidden), U32(streams)};
    return launch("hc_write_rows", (hidden + 255) / 256, streams, m, 256, 0, stream, a);
}

}   // extern "C"
