// The C entry points of the checkpoint readers, and the staging of one MoE layer from a GGUF or an EXL3 safetensors
// checkpoint into the device layout sz_session_set_layer takes: expert e's [gate | up | down] at e * stride, then the shared
// expert's three, the router and the shared expert's gate.  Where each slice lies in the files follows
// Model::expert_file_range (crates/shadowzero-model/src/forward.rs:477-486): a GGUF stacks the experts of a fused tensor
// evenly, an EXL3 checkpoint has one blob per expert and projection.
//
// Staging reads with pread on several threads into one of two pinned buffers while the other one's host-to-device
// copies run: the disk (or page cache), the host memory copy and the PCIe transfer overlap.
#include <fcntl.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <memory>
#include <mutex>
#include <thread>

#include "sz_formats.hpp"

using namespace sz;

namespace {

int copy_out(const std::string& s, char* buf, uint64_t len) {
    if (!buf || len < s.size() + 1) return fail("a buffer of " + std::to_string(len) + " bytes for " + std::to_string(s.size() + 1));
    std::memcpy(buf, s.c_str(), s.size() + 1);
    return 0;
}

void fill_info(const GgufTensor& t, sz_tensor_info* o) {
    std::memset(o, 0, sizeof *o);
    o->type = t.type;
    o->n_dims = (uint32_t) t.dims.size();
    for (size_t i = 0; i < t.dims.size(); i++) o->dims[i] = t.dims[i];
    o->shard = t.shard;
    o->has_layout = t.has_layout;
    o->offset = t.offset;
    o->nbytes_layout = t.layout;
    o->nbytes_span = t.span;
    o->nbytes = t.nbytes();
}

const GgufValue* kv_of(const sz_gguf* g, const char* key, bool arch) {
    if (!g || !key) return nullptr;
    return arch ? g->g.arch_key(key) : g->g.get(key);
}

int no_key(const char* key) { return fail(std::string("no key ") + (key ? key : "(null)") + " of that type"); }

}   // namespace

// ---- GGUF ---------------------------------------------------------------------------------------------------------------
extern "C" {

int32_t sz_type_info(uint32_t type, char* name, uint64_t len, uint64_t* block_elements, uint64_t* block_bytes) {
    clear_error();
    uint64_t be = 0, bb = 0;
    type_block(type, be, bb);
    if (block_elements) *block_elements = be;
    if (block_bytes) *block_bytes = bb;
    return name ? copy_out(type_name(type), name, len) : 0;
}

int32_t sz_gguf_shard_paths(const char* path, uint32_t i, char* buf, uint64_t len, uint32_t* count) {
    clear_error();
    if (!path) return fail("sz_gguf_shard_paths: null path");
    const std::vector<std::string> v = gguf_shard_paths(path);
    if (count) *count = (uint32_t) v.size();
    if (!buf) return 0;
    if (i >= v.size()) return fail("sz_gguf_shard_paths: shard " + std::to_string(i) + " of " + std::to_string(v.size()));
    return copy_out(v[i], buf, len);
}

int32_t sz_gguf_open(const char* path, sz_gguf** out) {
    clear_error();
    if (!path || !out) return fail("sz_gguf_open: null argument");
    std::unique_ptr<sz_gguf> g(new sz_gguf);
    if (gguf_open(path, g->g)) return 1;
    *out = g.release();
    return 0;
}

void sz_gguf_close(sz_gguf* g) { delete g; }

uint64_t sz_gguf_tensor_count(const sz_gguf* g) { return g ? g->g.tensors.size() : 0; }

int32_t sz_gguf_tensor_at(const sz_gguf* g, uint64_t i, char* name, uint64_t name_len, sz_tensor_info* info) {
    clear_error();
    if (!g || i >= g->g.tensors.size()) return fail("sz_gguf_tensor_at: no tensor " + std::to_string(i));
    if (info) fill_info(g->g.tensors[i], info);
    return name ? copy_out(g->g.tensors[i].name, name, name_len) : 0;
}

int32_t sz_gguf_tensor(const sz_gguf* g, const char* name, sz_tensor_info* info) {
    clear_error();
    const GgufTensor* t = g && name ? g->g.tensor(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (info) fill_info(*t, info);
    return 0;
}

uint64_t sz_gguf_tensor_bytes(const sz_gguf* g) {
    uint64_t n = 0;
    if (g)
        for (const GgufTensor& t : g->g.tensors) n += t.nbytes();
    return n;
}

uint32_t sz_gguf_shard_count(const sz_gguf* g) { return g ? (uint32_t) g->g.shards.size() : 0; }

int32_t sz_gguf_shard(const sz_gguf* g, uint32_t i, char* path, uint64_t path_len, uint32_t* version, uint64_t* file_len, uint64_t* data_start,
                      uint64_t* alignment) {
    clear_error();
    if (!g || i >= g->g.shards.size()) return fail("sz_gguf_shard: no shard " + std::to_string(i));
    const GgufShard& s = g->g.shards[i];
    if (version) *version = s.version;
    if (file_len) *file_len = s.file_len;
    if (data_start) *data_start = s.data_start;
    if (alignment) *alignment = s.alignment;
    return path ? copy_out(s.path, path, path_len) : 0;
}

uint64_t sz_gguf_kv_count(const sz_gguf* g) { return g ? g->g.kv.size() : 0; }

int32_t sz_gguf_kv_key(const sz_gguf* g, uint64_t i, char* buf, uint64_t len) {
    clear_error();
    if (!g || i >= g->g.kv.size()) return fail("sz_gguf_kv_key: no key " + std::to_string(i));
    auto it = g->g.kv.begin();
    std::advance(it, (long) i);
    return copy_out(it->first, buf, len);
}

int32_t sz_gguf_kv_type(const sz_gguf* g, const char* key, uint32_t* type, uint32_t* elem_type, uint64_t* count) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    if (!v) return no_key(key);
    if (type) *type = v->type;
    if (elem_type) *elem_type = v->type == 9 ? v->elem_type : 0;
    if (count) *count = v->type == 9 ? v->arr.size() : v->type == 8 ? v->s.size() : 1;
    return 0;
}

int32_t sz_gguf_kv_u64(const sz_gguf* g, const char* key, uint64_t* out) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    return v && out && v->as_u64(*out) ? 0 : no_key(key);
}

int32_t sz_gguf_arch_u64(const sz_gguf* g, const char* key, uint64_t* out) {
    clear_error();
    const GgufValue* v = kv_of(g, key, true);
    return v && out && v->as_u64(*out) ? 0 : no_key(key);
}

int32_t sz_gguf_kv_f64(const sz_gguf* g, const char* key, double* out) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    return v && out && v->as_f64(*out) ? 0 : no_key(key);
}

int32_t sz_gguf_kv_str(const sz_gguf* g, const char* key, char* buf, uint64_t len) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    if (!v || v->type != 8) return no_key(key);
    return copy_out(v->s, buf, len);
}

int32_t sz_gguf_kv_array_u64(const sz_gguf* g, const char* key, uint64_t i, uint64_t* out) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    if (!v || v->type != 9 || i >= v->arr.size() || !out) return no_key(key);
    if (v->arr[i].type == 7) return *out = v->arr[i].u, 0;   // a flag array (attention.recurrent_layers)
    return v->arr[i].as_u64(*out) ? 0 : no_key(key);
}

int32_t sz_gguf_kv_array_f64(const sz_gguf* g, const char* key, uint64_t i, double* out) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    if (!v || v->type != 9 || i >= v->arr.size() || !out) return no_key(key);
    return v->arr[i].as_f64(*out) ? 0 : no_key(key);
}

int32_t sz_gguf_kv_array_str(const sz_gguf* g, const char* key, uint64_t i, char* buf, uint64_t len) {
    clear_error();
    const GgufValue* v = kv_of(g, key, false);
    if (!v || v->type != 9 || i >= v->arr.size() || v->arr[i].type != 8) return no_key(key);
    return copy_out(v->arr[i].s, buf, len);
}

int64_t sz_gguf_block_index(const char* name) {
    if (!name || std::strncmp(name, "blk.", 4) != 0) return -1;
    const char* p = name + 4;
    if (*p == '+') p++;   // usize::from_str accepts a leading plus sign
    if (*p < '0' || *p > '9') return -1;
    uint64_t v = 0;
    for (; *p >= '0' && *p <= '9'; p++) {
        if (v > (uint64_t) INT64_MAX / 10 - 1) return -1;
        v = v * 10 + (uint64_t) (*p - '0');
    }
    return *p == '.' || *p == '\0' ? (int64_t) v : -1;
}

int32_t sz_gguf_read_tensor(const sz_gguf* g, const char* name, void* host, uint64_t cap) {
    clear_error();
    const GgufTensor* t = g && name ? g->g.tensor(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (cap < t->nbytes()) return fail(std::string(name) + ": " + std::to_string(t->nbytes()) + " bytes into " + std::to_string(cap));
    return pread_exact(g->g.shards[t->shard].path, t->offset, host, t->nbytes());
}

int32_t sz_gguf_expert_range(const sz_gguf* g, const char* name, uint64_t e, uint32_t* shard, uint64_t* offset, uint64_t* len) {
    clear_error();
    const GgufTensor* t = g && name ? g->g.tensor(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (t->dims.size() < 3 || t->dims[2] == 0) return fail(std::string(name) + ": not a fused expert tensor");
    if (e >= t->dims[2]) return fail(std::string(name) + ": expert " + std::to_string(e) + " of " + std::to_string(t->dims[2]));
    const uint64_t per = t->nbytes() / t->dims[2];
    if (shard) *shard = t->shard;
    if (offset) *offset = t->offset + e * per;
    if (len) *len = per;
    return 0;
}

// ---- safetensors and the EXL3 projection --------------------------------------------------------------------------------
int32_t sz_st_open(const char* const* paths, uint32_t n, sz_safetensors** out) {
    clear_error();
    if (!out || (n && !paths)) return fail("sz_st_open: null argument");
    std::unique_ptr<sz_safetensors> st(new sz_safetensors);
    for (uint32_t i = 0; i < n; i++)
        if (!paths[i] || st->st.add_file(paths[i])) return paths[i] ? 1 : fail("sz_st_open: null path");
    *out = st.release();
    return 0;
}

int32_t sz_st_open_dir(const char* dir, sz_safetensors** out) {
    clear_error();
    if (!dir || !out) return fail("sz_st_open_dir: null argument");
    std::unique_ptr<sz_safetensors> st(new sz_safetensors);
    if (st->st.add_dir(dir)) return 1;
    *out = st.release();
    return 0;
}

void sz_st_close(sz_safetensors* st) { delete st; }

uint64_t sz_st_tensor_count(const sz_safetensors* st) { return st ? st->st.tensors.size() : 0; }
uint32_t sz_st_file_count(const sz_safetensors* st) { return st ? (uint32_t) st->st.files.size() : 0; }

int32_t sz_st_file(const sz_safetensors* st, uint32_t i, char* buf, uint64_t len) {
    clear_error();
    if (!st || i >= st->st.files.size()) return fail("sz_st_file: no file " + std::to_string(i));
    return copy_out(st->st.files[i], buf, len);
}

static void fill_st(const StTensor& t, sz_st_info* o) {
    std::memset(o, 0, sizeof *o);
    std::strncpy(o->dtype, t.dtype.c_str(), sizeof o->dtype - 1);
    o->n_dims = (uint32_t) std::min<size_t>(t.shape.size(), 8);
    for (uint32_t i = 0; i < o->n_dims; i++) o->shape[i] = t.shape[i];
    o->file = t.file;
    o->start = t.start;
    o->end = t.end;
}

int32_t sz_st_tensor_at(const sz_safetensors* st, uint64_t i, char* name, uint64_t name_len, sz_st_info* info) {
    clear_error();
    if (!st || i >= st->st.tensors.size()) return fail("sz_st_tensor_at: no tensor " + std::to_string(i));
    auto it = st->st.tensors.begin();
    std::advance(it, (long) i);
    if (info) fill_st(it->second, info);
    return name ? copy_out(it->first, name, name_len) : 0;
}

int32_t sz_st_tensor(const sz_safetensors* st, const char* name, sz_st_info* info) {
    clear_error();
    const StTensor* t = st && name ? st->st.get(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (info) fill_st(*t, info);
    return 0;
}

int32_t sz_st_read(const sz_safetensors* st, const char* name, uint64_t off, uint64_t len, void* host) {
    clear_error();
    const StTensor* t = st && name ? st->st.get(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    return st->st.read_range(*t, off, len, host);
}

int32_t sz_exl3_shape(const sz_safetensors* st, const char* prefix, uint64_t* in_features, uint64_t* out_features, int32_t* type) {
    clear_error();
    if (!st || !prefix) return fail("sz_exl3_shape: null argument");
    Exl3Shape s;
    if (exl3_linear_shape(st->st, prefix, s)) return 1;
    if (in_features) *in_features = s.in_f;
    if (out_features) *out_features = s.out_f;
    if (type) *type = (int32_t) s.type;
    return 0;
}

int32_t sz_exl3_contiguous(const sz_safetensors* st, const char* prefix, uint32_t* file, uint64_t* offset, uint64_t* len) {
    clear_error();
    if (!st || !prefix) return fail("sz_exl3_contiguous: null argument");
    uint32_t f;
    uint64_t o, l;
    if (!exl3_contiguous(st->st, prefix, f, o, l)) return fail(std::string(prefix) + ": its tensors are not one range of a file");
    if (file) *file = f;
    if (offset) *offset = o;
    if (len) *len = l;
    return 0;
}

uint64_t sz_exl3_blob_len(uint64_t in_features, uint64_t out_features, int32_t type) {
    const bool half = type >= 1031 && type <= 1033;
    const uint32_t bits = half ? type - 1030 : type > 1000 ? (uint32_t) (type - 1000) % 10 : 0;
    return bits ? exl3_blob_len(in_features, out_features, bits, half) : 0;
}

int32_t sz_exl3_read_blob(const sz_safetensors* st, const char* prefix, void* host, uint64_t cap) {
    clear_error();
    if (!st || !prefix || !host) return fail("sz_exl3_read_blob: null argument");
    return exl3_read_blob(st->st, prefix, host, cap);
}

}   // extern "C"

// ---- staging ----------------------------------------------------------------------------------------------------------
namespace {

struct Piece {
    uint32_t file = 0;         // index into the stager's file list
    uint64_t file_off = 0, len = 0, dev_off = 0;
    std::string blob_prefix;   // not empty: an EXL3 projection put together from its tensors (exl3_read_blob), len = its blob's
};

constexpr uint64_t CHUNK = 64ull << 20;      // a buffer, and the longest piece (longer file ranges are cut)
constexpr uint64_t ROUND = 16ull << 20;      // file bytes a round aims at: short rounds start the first copy early (47 GB/s measured from the page cache; 41 at 64 MiB)
constexpr uint64_t TABLE = 1ull << 20;       // the head of a buffer: the round's piece table (3 u64 a piece)

struct Staging {
    std::mutex mu;             // one staging call at a time: the buffers are the process's
    void* host[2] = {nullptr, nullptr};   // pinned
    void* dev[2] = {nullptr, nullptr};
    void* ev[2] = {nullptr, nullptr};
};
Staging& staging() {
    static Staging p;
    return p;
}

// reads the pieces [a, b) into base (piece i at offs[i]) on up to 8 threads; 0 or fail(first error)
int fill(const std::vector<std::string>& files, const std::vector<int>& fds, const SafeTensors* st, const std::vector<Piece>& ps, size_t a, size_t b,
         const std::vector<uint64_t>& offs, uint8_t* base) {
    const size_t nt = std::min<size_t>(8, b - a);
    std::vector<std::string> errs(nt);
    auto work = [&](size_t t) {
        for (size_t i = a + t; i < b; i += nt) {
            const Piece& p = ps[i];
            uint8_t* dst = base + offs[i - a];
            if (!p.blob_prefix.empty()) {
                if (exl3_read_blob(*st, p.blob_prefix, dst, p.len)) return (void) (errs[t] = sz_last_error());
                continue;
            }
            uint64_t done = 0;
            while (done < p.len) {
                const ssize_t n = ::pread(fds[p.file], dst + done, p.len - done, (off_t) (p.file_off + done));
                if (n < 0 && errno == EINTR) continue;
                if (n <= 0) return (void) (errs[t] = files[p.file] + ": " + (n < 0 ? std::strerror(errno) : "failed to fill whole buffer"));
                done += (uint64_t) n;
            }
        }
    };
    std::vector<std::thread> th;
    for (size_t t = 1; t < nt; t++) th.emplace_back(work, t);
    work(0);
    for (auto& t : th) t.join();
    for (const std::string& e : errs)
        if (!e.empty()) return fail(e);
    return 0;
}

// Every round: the next pieces (about ROUND bytes) are read into a pinned buffer behind their table, the buffer goes to the
// device as ONE copy (thousands of expert-sized copies would cost more in launches than in bytes), and a kernel moves the pieces
// to their places.  The other buffer is being filled meanwhile.
int stage(const std::vector<std::string>& files, const SafeTensors* st, std::vector<Piece> ps, uint64_t dev, uint64_t stream) {
    if (ensure_init()) return 1;
    // pieces larger than a round are cut (file ranges only: a projection's blob is far smaller)
    std::vector<Piece> cut;
    for (Piece& p : ps) {
        if (!p.blob_prefix.empty() && p.len > CHUNK) return fail(p.blob_prefix + ": a blob of " + std::to_string(p.len) + " bytes");
        for (uint64_t o = 0; o < p.len; o += CHUNK) {
            Piece q = p;
            q.file_off = p.file_off + o;
            q.dev_off = p.dev_off + o;
            q.len = std::min(CHUNK, p.len - o);
            cut.push_back(std::move(q));
        }
    }
    std::vector<int> fds(files.size(), -1);
    auto close_all = [&]() {
        for (int fd : fds)
            if (fd >= 0) ::close(fd);
    };
    for (const Piece& p : cut) {
        if (!p.blob_prefix.empty() || fds[p.file] >= 0) continue;
        fds[p.file] = ::open(files[p.file].c_str(), O_RDONLY | O_CLOEXEC);
        if (fds[p.file] < 0) {
            const std::string why = std::strerror(errno);
            close_all();
            return fail(files[p.file] + ": " + why);
        }
    }
    Staging& S = staging();
    std::lock_guard<std::mutex> lock(S.mu);
    HipApi& h = hip();
    for (int i = 0; i < 2; i++) {
        if (!S.host[i] && hip_check(h.hipHostMalloc(&S.host[i], TABLE + CHUNK, 0), "hipHostMalloc")) return close_all(), 1;
        if (!S.dev[i] && hip_check(h.hipMalloc(&S.dev[i], TABLE + CHUNK), "hipMalloc")) return close_all(), 1;
        if (!S.ev[i] && hip_check(h.hipEventCreate(&S.ev[i]), "hipEventCreate")) return close_all(), 1;
    }
    int rc = 0;
    size_t a = 0;
    for (uint32_t round = 0; a < cut.size() && !rc; round++) {
        std::vector<uint64_t> offs;   // of each piece in the buffer, behind the table, at 256-byte boundaries
        uint64_t used = 0, longest = 0;
        size_t b = a;
        while (b < cut.size() && (b == a || used + cut[b].len <= ROUND) && (b - a + 1) * 24 <= TABLE) {
            offs.push_back(TABLE + used);
            used = (used + cut[b].len + 255) & ~255ull;
            longest = std::max(longest, cut[b].len);
            b++;
        }
        const int k = round & 1;
        uint8_t* host = (uint8_t*) S.host[k];
        if (round >= 2) rc = hip_check(h.hipEventSynchronize(S.ev[k]), "hipEventSynchronize");   // the buffer's last copy has left it
        if (!rc) rc = fill(files, fds, st, cut, a, b, offs, host);
        if (rc) break;
        uint64_t* table = (uint64_t*) host;
        for (size_t i = a; i < b; i++) {
            table[3 * (i - a)] = offs[i - a];
            table[3 * (i - a) + 1] = cut[i].dev_off;
            table[3 * (i - a) + 2] = cut[i].len;
        }
        rc = hip_check(h.hipMemcpyHtoDAsync(S.dev[k], host, TABLE + used, (hipStream_t) stream), "hipMemcpyHtoDAsync");
        if (!rc) rc = hip_check(h.hipEventRecord(S.ev[k], (hipStream_t) stream), "hipEventRecord");
        if (!rc) {
            const sz_arg args[] = {P((uint64_t) S.dev[k]), P(dev), P((uint64_t) S.dev[k]), U32((uint32_t) (b - a))};
            rc = launch("scatter_pieces", (uint32_t) ((longest + 65535) >> 16), (uint32_t) (b - a), 1, 256, 0, stream, args);
        }
        a = b;
    }
    // the buffers belong to the next call once this one returns: every copy and kernel has to be through with them
    const std::string err = rc ? sz_last_error() : "";
    const int rs = hip_check(h.hipStreamSynchronize((hipStream_t) stream), "hipStreamSynchronize");
    close_all();
    if (rc) return fail(err);
    return rs;
}

uint64_t up256(uint64_t v) { return (v + 255) & ~255ull; }

int dense_type_of(const std::string& dtype) { return dtype == "F32" ? SZ_TYPE_F32 : dtype == "F16" ? SZ_TYPE_F16 : dtype == "BF16" ? SZ_TYPE_BF16 : -1; }

// the layout from the sizes: experts, the shared expert (shared_down_bytes: its down projection, 0 without one), the router,
// the shared expert's gate.  An expert's projections lie L.gap apart and the first one `lead` bytes past a 256-byte
// boundary (sz_layer_spacing: what puts the rows of an EXL3 trellis on the 128-byte lines of memory; 0 and 0 for a GGUF).
void place(sz_layer_layout& L, uint64_t shared_down_bytes, uint64_t router_bytes, uint64_t gate_bytes) {
    uint32_t lead = 0, gap = 0;
    sz_layer_spacing(L.type, L.hidden, L.ff, &lead, &gap);
    L.gap = gap;
    L.experts_offset = lead;
    L.stride = up256(2 * (L.gate_up_bytes + gap) + L.down_bytes);
    uint64_t at = up256(lead + (uint64_t) L.n_expert * L.stride);
    L.shared_offset = at + lead;
    const uint64_t shared_bytes = shared_down_bytes ? 2 * (L.shared_gate_up_bytes + gap) + shared_down_bytes : 0;
    at = up256(L.shared_offset + shared_bytes);
    L.router_offset = at;
    at = up256(at + router_bytes);
    L.gate_offset = at;
    L.bytes = up256(at + gate_bytes);
}

struct GgufLayer {
    const GgufTensor *e[3] = {}, *sh[3] = {}, *router = nullptr, *gate = nullptr;
};

int gguf_layer(const sz_gguf* g, uint32_t layer, sz_layer_layout& L, GgufLayer& T) {
    if (!g) return fail("null GGUF handle");
    const std::string p = "blk." + std::to_string(layer) + ".";
    static const char* const EN[3] = {"ffn_gate_exps.weight", "ffn_up_exps.weight", "ffn_down_exps.weight"};
    static const char* const SN[3] = {"ffn_gate_shexp.weight", "ffn_up_shexp.weight", "ffn_down_shexp.weight"};
    for (int i = 0; i < 3; i++) {
        T.e[i] = g->g.tensor(p + EN[i]);
        if (!T.e[i]) return fail("no tensor " + p + EN[i]);
        if (T.e[i]->dims.size() != 3) return fail(p + EN[i] + ": not a fused expert tensor [in, out, n_expert]");
    }
    std::memset(&L, 0, sizeof L);
    const GgufTensor &ga = *T.e[0], &up = *T.e[1], &dn = *T.e[2];
    if (up.dims != ga.dims || dn.dims[0] != ga.dims[1] || dn.dims[1] != ga.dims[0] || dn.dims[2] != ga.dims[2] || ga.dims[2] == 0)
        return fail(p + "ffn_*_exps: the three projections' shapes do not fit together");
    if (up.type != ga.type || dn.type != ga.type)
        return fail(p + "ffn_*_exps: projections of types " + type_name(ga.type) + ", " + type_name(up.type) + ", " + type_name(dn.type) + " (one type a layer is staged)");
    L.type = (int32_t) ga.type;
    L.n_expert = (uint32_t) ga.dims[2];
    L.hidden = ga.dims[0];
    L.ff = ga.dims[1];
    L.gate_up_bytes = ga.nbytes() / ga.dims[2];
    L.down_bytes = dn.nbytes() / dn.dims[2];
    if (up.nbytes() / up.dims[2] != L.gate_up_bytes) return fail(p + "ffn_up_exps.weight: its experts' size differs from the gate's");
    L.shared_type = L.router_type = L.gate_type = -1;
    uint64_t shared_bytes = 0, router_bytes = 0, gate_bytes = 0;
    T.sh[0] = g->g.tensor(p + SN[0]);
    if (T.sh[0]) {
        for (int i = 1; i < 3; i++)
            if (!(T.sh[i] = g->g.tensor(p + SN[i]))) return fail("no tensor " + p + SN[i]);
        const GgufTensor &sg = *T.sh[0], &su = *T.sh[1], &sd = *T.sh[2];
        if (sg.dims.size() != 2 || su.dims != sg.dims || sd.dims.size() != 2 || sd.dims[0] != sg.dims[1] || sd.dims[1] != sg.dims[0] || sg.dims[0] != L.hidden)
            return fail(p + "ffn_*_shexp: the three projections' shapes do not fit together");
        if (sg.dims[1] != L.ff) return fail(p + "ffn_gate_shexp.weight: a shared expert of width " + std::to_string(sg.dims[1]) + " beside experts of " + std::to_string(L.ff));
        if (su.type != sg.type || sd.type != sg.type) return fail(p + "ffn_*_shexp: projections of different types");
        L.shared_type = (int32_t) sg.type;
        L.shared_gate_up_bytes = sg.nbytes();
        if (su.nbytes() != sg.nbytes()) return fail(p + "ffn_up_shexp.weight: its size differs from the gate's");
        shared_bytes = sd.nbytes();   // (the down projection's: place() adds the other two)
    }
    T.router = g->g.tensor(p + "ffn_gate_inp.weight");
    if (T.router) {
        const GgufTensor& r = *T.router;
        if (r.dims.size() != 2 || r.dims[0] != L.hidden || r.dims[1] != L.n_expert) return fail(p + "ffn_gate_inp.weight: not [hidden, n_expert]");
        L.router_type = (int32_t) r.type;
        router_bytes = r.nbytes();
    }
    T.gate = g->g.tensor(p + "ffn_gate_inp_shexp.weight");
    if (T.gate) {
        uint64_t n = 1;
        for (uint64_t d : T.gate->dims) n *= d;
        if (n != L.hidden) return fail(p + "ffn_gate_inp_shexp.weight: not [hidden]");
        L.gate_type = (int32_t) T.gate->type;
        gate_bytes = T.gate->nbytes();
    }
    place(L, shared_bytes, router_bytes, gate_bytes);
    return 0;
}

struct Exl3Layer {
    std::vector<std::string> expert[3];   // prefixes, one a projection and expert
    std::string shared[3];
    const StTensor *router = nullptr, *gate = nullptr;
};

int exl3_layer(const sz_safetensors* st, uint32_t layer, uint32_t n_expert, sz_layer_layout& L, Exl3Layer& T) {
    if (!st) return fail("null safetensors handle");
    const std::string p = "model.language_model.layers." + std::to_string(layer) + ".mlp.";
    static const char* const PN[3] = {"gate_proj", "up_proj", "down_proj"};
    if (n_expert == 0)   // not given: as many as the checkpoint has
        while (st->st.get(p + "experts." + std::to_string(n_expert) + ".gate_proj.trellis")) n_expert++;
    if (n_expert == 0) return fail("no tensor " + p + "experts.0.gate_proj.trellis");
    std::memset(&L, 0, sizeof L);
    Exl3Shape first[3];
    for (int i = 0; i < 3; i++) {
        for (uint32_t e = 0; e < n_expert; e++) {
            const std::string pe = p + "experts." + std::to_string(e) + "." + PN[i];
            Exl3Shape s;
            if (exl3_linear_shape(st->st, pe, s)) return 1;
            if (e == 0) first[i] = s;
            const Exl3Shape& f = first[i];
            if (s.in_f != f.in_f || s.out_f != f.out_f || s.type != f.type)
                return fail(pe + ": " + std::to_string(s.in_f) + " x " + std::to_string(s.out_f) + " " + type_name(s.type) + ", but expert 0 of the layer is " +
                            std::to_string(f.in_f) + " x " + std::to_string(f.out_f) + " " + type_name(f.type));
            T.expert[i].push_back(pe);
        }
    }
    if (first[1].in_f != first[0].in_f || first[1].out_f != first[0].out_f || first[2].in_f != first[0].out_f || first[2].out_f != first[0].in_f)
        return fail(p + "experts: the three projections' shapes do not fit together");
    if (first[1].type != first[0].type || first[2].type != first[0].type)
        return fail(p + "experts: projections of types " + type_name(first[0].type) + ", " + type_name(first[1].type) + ", " + type_name(first[2].type) + " (one type a layer is staged)");
    L.type = (int32_t) first[0].type;
    L.n_expert = n_expert;
    L.hidden = first[0].in_f;
    L.ff = first[0].out_f;
    L.gate_up_bytes = exl3_blob_len(L.hidden, L.ff, first[0].bits, first[0].half);
    L.down_bytes = exl3_blob_len(L.ff, L.hidden, first[0].bits, first[0].half);
    L.shared_type = L.router_type = L.gate_type = -1;
    uint64_t shared_bytes = 0, router_bytes = 0, gate_bytes = 0;
    if (st->st.get(p + "shared_expert.gate_proj.trellis")) {
        Exl3Shape s[3];
        for (int i = 0; i < 3; i++) {
            T.shared[i] = p + "shared_expert." + PN[i];
            if (exl3_linear_shape(st->st, T.shared[i], s[i])) return 1;
        }
        if (s[0].in_f != L.hidden || s[1].in_f != L.hidden || s[1].out_f != s[0].out_f || s[2].in_f != s[0].out_f || s[2].out_f != L.hidden)
            return fail(p + "shared_expert: the three projections' shapes do not fit together");
        if (s[0].out_f != L.ff) return fail(p + "shared_expert: width " + std::to_string(s[0].out_f) + " beside experts of " + std::to_string(L.ff));
        if (s[1].type != s[0].type || s[2].type != s[0].type) return fail(p + "shared_expert: projections of different types");
        L.shared_type = (int32_t) s[0].type;
        L.shared_gate_up_bytes = exl3_blob_len(L.hidden, L.ff, s[0].bits, s[0].half);
        shared_bytes = exl3_blob_len(L.ff, L.hidden, s[0].bits, s[0].half);   // (the down projection's: place() adds the other two)
    }
    T.router = st->st.get(p + "gate.weight");
    if (T.router) {
        const StTensor& r = *T.router;
        L.router_type = dense_type_of(r.dtype);
        if (L.router_type < 0) return fail(p + "gate.weight: raw " + r.dtype);
        if (r.shape.size() != 2 || r.shape[0] != n_expert || r.shape[1] != L.hidden) return fail(p + "gate.weight: not [n_expert, hidden]");
        router_bytes = r.end - r.start;
    }
    T.gate = st->st.get(p + "shared_expert_gate.weight");
    if (T.gate) {
        uint64_t n = 1;
        for (uint64_t d : T.gate->shape) n *= d;
        L.gate_type = dense_type_of(T.gate->dtype);
        if (L.gate_type < 0) return fail(p + "shared_expert_gate.weight: raw " + T.gate->dtype);
        if (n != L.hidden) return fail(p + "shared_expert_gate.weight: not [hidden]");
        gate_bytes = T.gate->end - T.gate->start;
    }
    place(L, shared_bytes, router_bytes, gate_bytes);
    return 0;
}

}   // namespace

extern "C" {

int32_t sz_gguf_layer_layout(const sz_gguf* g, uint32_t layer, sz_layer_layout* out) {
    clear_error();
    GgufLayer T;
    sz_layer_layout L;
    if (!out) return fail("sz_gguf_layer_layout: null argument");
    if (gguf_layer(g, layer, L, T)) return 1;
    *out = L;
    return 0;
}

int32_t sz_gguf_stage_layer(const sz_gguf* g, uint32_t layer, uint64_t dev, uint64_t cap, uint64_t stream) {
    clear_error();
    GgufLayer T;
    sz_layer_layout L;
    if (gguf_layer(g, layer, L, T)) return 1;
    if (cap < L.bytes) return fail("sz_gguf_stage_layer: " + std::to_string(L.bytes) + " bytes into " + std::to_string(cap));
    if (dev & 255) return fail("sz_gguf_stage_layer: the device buffer must be 256-byte aligned");
    std::vector<std::string> files;
    for (const GgufShard& s : g->g.shards) files.push_back(s.path);
    std::vector<Piece> ps;
    const uint64_t part_off[3] = {L.experts_offset, L.experts_offset + L.gate_up_bytes + L.gap, L.experts_offset + 2 * (L.gate_up_bytes + L.gap)};
    // in file order (projection, then expert): the reads of a fused tensor are sequential
    for (int i = 0; i < 3; i++) {
        const uint64_t per = T.e[i]->nbytes() / L.n_expert;
        for (uint32_t e = 0; e < L.n_expert; e++) {
            Piece q;
            q.file = T.e[i]->shard;
            q.file_off = T.e[i]->offset + e * per;
            q.len = per;
            q.dev_off = e * L.stride + part_off[i];
            ps.push_back(std::move(q));
        }
    }
    auto whole = [&](const GgufTensor* t, uint64_t at) {
        Piece q;
        q.file = t->shard;
        q.file_off = t->offset;
        q.len = t->nbytes();
        q.dev_off = at;
        ps.push_back(std::move(q));
    };
    if (T.sh[0]) {
        whole(T.sh[0], L.shared_offset);
        whole(T.sh[1], L.shared_offset + L.shared_gate_up_bytes + L.gap);
        whole(T.sh[2], L.shared_offset + 2 * (L.shared_gate_up_bytes + L.gap));
    }
    if (T.router) whole(T.router, L.router_offset);
    if (T.gate) whole(T.gate, L.gate_offset);
    return stage(files, nullptr, std::move(ps), dev, stream);
}

int32_t sz_exl3_layer_layout(const sz_safetensors* st, uint32_t layer, uint32_t n_expert, sz_layer_layout* out) {
    clear_error();
    Exl3Layer T;
    sz_layer_layout L;
    if (!out) return fail("sz_exl3_layer_layout: null argument");
    if (exl3_layer(st, layer, n_expert, L, T)) return 1;
    *out = L;
    return 0;
}

int32_t sz_exl3_stage_layer(const sz_safetensors* st, uint32_t layer, uint32_t n_expert, uint64_t dev, uint64_t cap, uint64_t stream) {
    clear_error();
    Exl3Layer T;
    sz_layer_layout L;
    if (exl3_layer(st, layer, n_expert, L, T)) return 1;
    if (cap < L.bytes) return fail("sz_exl3_stage_layer: " + std::to_string(L.bytes) + " bytes into " + std::to_string(cap));
    if (dev & 255) return fail("sz_exl3_stage_layer: the device buffer must be 256-byte aligned");
    std::vector<Piece> ps;
    auto blob = [&](const std::string& prefix, uint64_t len, uint64_t at) {
        Piece q;
        q.len = len;
        q.dev_off = at;
        uint32_t f;
        uint64_t o, l;
        if (exl3_contiguous(st->st, prefix, f, o, l) && l == len) {   // one range of a file, as the reference's expert table lists it (exl3_model.rs:291-302)
            q.file = f;
            q.file_off = o;
        } else {
            q.blob_prefix = prefix;                                    // put together from its tensors (Exl3Extra::bytes, exl3_model.rs:432)
        }
        ps.push_back(std::move(q));
    };
    for (uint32_t e = 0; e < L.n_expert; e++) {
        const uint64_t at = L.experts_offset + e * L.stride, pitch = L.gate_up_bytes + L.gap;
        blob(T.expert[0][e], L.gate_up_bytes, at);
        blob(T.expert[1][e], L.gate_up_bytes, at + pitch);
        blob(T.expert[2][e], L.down_bytes, at + 2 * pitch);
    }
    if (!T.shared[0].empty()) {
        const uint64_t sgu = L.shared_gate_up_bytes, pitch = sgu + L.gap;
        blob(T.shared[0], sgu, L.shared_offset);
        blob(T.shared[1], sgu, L.shared_offset + pitch);
        blob(T.shared[2], sz_exl3_blob_len(L.ff, L.hidden, L.shared_type), L.shared_offset + 2 * pitch);
    }
    auto whole = [&](const StTensor* t, uint64_t at) {
        Piece q;
        q.file = t->file;
        q.file_off = t->start;
        q.len = t->end - t->start;
        q.dev_off = at;
        ps.push_back(std::move(q));
    };
    if (T.router) whole(T.router, L.router_offset);
    if (T.gate) whole(T.gate, L.gate_offset);
    // the file reads sorted by place in the files: scattered blobs become forward reads
    std::stable_sort(ps.begin(), ps.end(), [](const Piece& a, const Piece& b) {
        if (a.blob_prefix.empty() != b.blob_prefix.empty()) return a.blob_prefix.empty();
        return a.file != b.file ? a.file < b.file : a.file_off < b.file_off;
    });
    return stage(st->st.files, &st->st, std::move(ps), dev, stream);
}

int32_t sz_gguf_stage_tensor(const sz_gguf* g, const char* name, uint64_t dev, uint64_t cap, uint64_t stream) {
    clear_error();
    const GgufTensor* t = g && name ? g->g.tensor(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (cap < t->nbytes()) return fail(std::string(name) + ": " + std::to_string(t->nbytes()) + " bytes into " + std::to_string(cap));
    std::vector<std::string> files;
    for (const GgufShard& sh : g->g.shards) files.push_back(sh.path);
    Piece q;
    q.file = t->shard;
    q.file_off = t->offset;
    q.len = t->nbytes();
    return stage(files, nullptr, {q}, dev, stream);
}

int32_t sz_st_stage_tensor(const sz_safetensors* st, const char* name, uint64_t dev, uint64_t cap, uint64_t stream) {
    clear_error();
    const StTensor* t = st && name ? st->st.get(name) : nullptr;
    if (!t) return fail(std::string("no tensor ") + (name ? name : "(null)"));
    if (cap < t->end - t->start) return fail(std::string(name) + ": " + std::to_string(t->end - t->start) + " bytes into " + std::to_string(cap));
    Piece q;
    q.file = t->file;
    q.file_off = t->start;
    q.len = t->end - t->start;
    return stage(st->st.files, &st->st, {q}, dev, stream);
}

int32_t sz_exl3_stage_blob(const sz_safetensors* st, const char* prefix, uint64_t dev, uint64_t cap, uint64_t stream) {
    clear_error();
    if (!st || !prefix) return fail("sz_exl3_stage_blob: null argument");
    Exl3Shape sh;
    if (exl3_linear_shape(st->st, prefix, sh)) return 1;
    const uint64_t len = exl3_blob_len(sh.in_f, sh.out_f, sh.bits, sh.half);
    if (cap < len) return fail(std::string(prefix) + ": a blob of " + std::to_string(len) + " bytes into " + std::to_string(cap));
    Piece q;
    q.len = len;
    uint32_t f;
    uint64_t o, l;
    if (exl3_contiguous(st->st, prefix, f, o, l) && l == len) {
        q.file = f;
        q.file_off = o;
    } else {
        q.blob_prefix = prefix;   // put together from its tensors (up to a staging buffer's 64 MiB)
    }
    return stage(st->st.files, &st->st, {q}, dev, stream);
}

}   // extern "C"
