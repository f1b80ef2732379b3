// The kernel programs: sources shipped beside the library, compiled ahead of time (hipcc --genco) or at run time (hiprtc)
// into a SHA-256-keyed code-object cache, loaded with hipModuleLoadData, and launched through a registry check.  The
// counterpart of crates/shadowzero-cuda/src/{kernels,nvrtc,sha256}.rs.
#include <dlfcn.h>
#include <sys/stat.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>
#include <unordered_map>

#include "sz_internal.hpp"

namespace sz {

#include "registry.inc"

// ---- SHA-256 (FIPS 180-4) ----------------------------------------------------------------------------------------
static const uint32_t K256[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
    0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
    0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
    0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
    0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
    0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

std::string sha256_hex(const std::string& data) {
    uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    std::string msg = data;
    const uint64_t bits = (uint64_t) data.size() * 8;
    msg.push_back((char) 0x80);
    while (msg.size() % 64 != 56) msg.push_back(0);
    for (int i = 7; i >= 0; i--) msg.push_back((char) (bits >> (8 * i)));
    auto rotr = [](uint32_t x, int n) { return (x >> n) | (x << (32 - n)); };
    for (size_t off = 0; off < msg.size(); off += 64) {
        uint32_t w[64];
        for (int i = 0; i < 16; i++) {
            const unsigned char* p = (const unsigned char*) msg.data() + off + 4 * i;
            w[i] = (uint32_t) p[0] << 24 | (uint32_t) p[1] << 16 | (uint32_t) p[2] << 8 | p[3];
        }
        for (int i = 16; i < 64; i++) {
            const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
            const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
            w[i] = w[i - 16] + s0 + w[i - 7] + s1;
        }
        uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
        for (int i = 0; i < 64; i++) {
            const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + K256[i] + w[i];
            const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
            hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
        }
        h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
    }
    char out[65];
    for (int i = 0; i < 8; i++) std::snprintf(out + 8 * i, 9, "%08x", h[i]);
    return std::string(out, 64);
}

// ---- registry -----------------------------------------------------------------------------------------------------
int entry_count() { return (int) (sizeof(SZ_ENTRIES) / sizeof(SZ_ENTRIES[0])); }
const SzEntry* entry(int i) { return i >= 0 && i < entry_count() ? &SZ_ENTRIES[i] : nullptr; }
const SzEntry* find_entry(const char* name) {
    static std::unordered_map<std::string, const SzEntry*> map;
    static std::once_flag once;
    std::call_once(once, [] {
        for (int i = 0; i < entry_count(); i++) map[SZ_ENTRIES[i].name] = &SZ_ENTRIES[i];
    });
    auto it = map.find(name);
    return it == map.end() ? nullptr : it->second;
}
int file_count() { return (int) (sizeof(SZ_FILES) / sizeof(SZ_FILES[0])); }
const char* file_name(int i) { return i >= 0 && i < file_count() ? SZ_FILES[i] : nullptr; }
static int file_index(const char* file) {
    for (int i = 0; i < file_count(); i++)
        if (!std::strcmp(SZ_FILES[i], file)) return i;
    return -1;
}

// ---- sources and cache ----------------------------------------------------------------------------------------------
static std::string lib_dir() {
    Dl_info info;
    if (dladdr((void*) &lib_dir, &info) && info.dli_fname) {
        std::string p = info.dli_fname;
        const size_t s = p.rfind('/');
        return s == std::string::npos ? "." : p.substr(0, s);
    }
    return ".";
}
std::string kernel_dir() {
    if (const char* e = std::getenv("SHADOWZERO_KERNEL_DIR")) return e;
    return lib_dir() + "/kernels";
}
std::string cache_dir() {
    if (const char* e = std::getenv("SHADOWZERO_KERNEL_CACHE")) return e;
    return kernel_dir() + "/cache";
}
// No fast-math; contraction off so the dequantizers keep the reference's two roundings (nvrtc.rs:149-156); packed FP32
// instructions off.
const char* compile_options() { return "-O3 -std=c++17 -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops"; }

static bool read_file(const std::string& path, std::string& out) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::ostringstream ss;
    ss << f.rdbuf();
    out = ss.str();
    return true;
}

int program_source(const char* file, std::string& out) {
    const int fi = file_index(file);
    if (fi < 0) return fail(std::string(file) + " is not a registered kernel file");
    const std::string dir = kernel_dir();
    std::string part;
    out.clear();
    auto add = [&](const std::string& name) -> bool {
        if (!read_file(dir + "/" + name, part)) return false;
        out += "#line 1 \"" + name + "\"\n" + part + "\n";
        return true;
    };
    if (!add("prelude.hip.h")) return fail("cannot read " + dir + "/prelude.hip.h");
    for (int h = 0; SZ_FILE_HEADERS[fi][h]; h++)
        if (!add(SZ_FILE_HEADERS[fi][h])) return fail("cannot read " + dir + "/" + SZ_FILE_HEADERS[fi][h]);
    if (!add(file)) return fail("cannot read " + dir + "/" + file);
    return 0;
}

// The options a kernel file asks the ahead-of-time compiler for on top of compile_options(): its `// hipcc: <options>` lines,
// joined by spaces (preferences of code generation; the run-time compiler does not get them).
static std::string extra_options(const std::string& src) {
    std::string out;
    size_t pos = 0;
    const std::string tag = "// hipcc: ";
    while (pos < src.size()) {
        size_t end = src.find('\n', pos);
        if (end == std::string::npos) end = src.size();
        if (src.compare(pos, tag.size(), tag) == 0) {
            if (!out.empty()) out += ' ';
            out += src.substr(pos + tag.size(), end - pos - tag.size());
        }
        pos = end + 1;
    }
    while (!out.empty() && (out.back() == ' ' || out.back() == '\r')) out.pop_back();
    return out;
}

// The cache key of a kernel file's code object: SHA-256 over the assembled source, the options, the target and HOW it was
// built (nvrtc.rs:185-194 hashes source + options + target).  An object compiled ahead of time by hipcc (with the file's extra
// options) and one compiled at run time by hiprtc (without) are different binaries and get different names, so the one
// can never stand in for the other.
int cache_key(const char* file, std::string& hex, bool run_time) {
    std::string src;
    if (program_source(file, src)) return 1;
    const std::string opts = run_time ? std::string(compile_options()) : aot_options_of(src);
    hex = sha256_hex(src + '\0' + opts + '\0' + "gfx950" + '\0' + (run_time ? "hiprtc" : "hipcc"));
    return 0;
}
std::string aot_options_of(const std::string& src) {
    const std::string extra = extra_options(src);
    return extra.empty() ? std::string(compile_options()) : std::string(compile_options()) + " " + extra;
}

// ---- loading and launching ----------------------------------------------------------------------------------------
struct Loaded {
    hipModule_t module = nullptr;
    bool tried = false;
    std::string error;
};
static std::vector<Loaded> g_modules;
static std::unordered_map<std::string, hipFunction_t> g_functions;
static std::mutex g_mutex;
static bool g_init = false;
static int g_device = -1;
static std::atomic<uint64_t> g_launches{0};

// per-launch event pairs while sz_ktime_begin is in force (kernels.rs:570-583)
struct Timed {
    const char* name;
    hipEvent_t a, b;
};
static bool g_ktime = false;
static std::string g_ktime_prefix;
static std::vector<Timed> g_timed;
static int g_capturing = 0;   // launches recorded into a stream capture are not timed

bool initialized() { return g_init; }
int ensure_init() { return g_init ? 0 : fail("sz_init has not been called (or failed)"); }

static int load_file(int fi) {
    Loaded& L = g_modules[fi];
    if (L.module) return 0;
    if (L.tried) return fail(L.error);
    L.tried = true;
    const char* file = SZ_FILES[fi];
    std::string key, rkey;
    if (cache_key(file, key, false) || cache_key(file, rkey, true)) {
        L.error = sz_last_error();
        return 1;
    }
    // the object built ahead of time first, then one an earlier run compiled with hiprtc
    std::string path = cache_dir() + "/" + key + ".hsaco";
    std::string image;
    if (!read_file(path, image)) path = cache_dir() + "/" + rkey + ".hsaco";
    if (image.empty() && !read_file(path, image)) {
        // miss: compile at run time and fill the cache (tmp + rename; a failed write is tolerated, nvrtc.rs:247-254)
        std::string src, log;
        std::vector<char> code;
        if (program_source(file, src) || rtc_compile(file, src, code, log)) {
            L.error = std::string("no cached code object ") + path + " and the run-time compile failed: " + sz_last_error();
            return fail(L.error);
        }
        image.assign(code.begin(), code.end());
        ::mkdir(cache_dir().c_str(), 0755);
        const std::string tmp = path + ".tmp";
        std::ofstream f(tmp, std::ios::binary);
        if (f) {
            f.write(image.data(), (std::streamsize) image.size());
            f.close();
            if (std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
        }
    }
    if (hip_check(hip().hipModuleLoadData(&L.module, image.data()), (std::string("hipModuleLoadData(") + file + ")").c_str())) {
        L.error = sz_last_error();
        L.module = nullptr;
        return 1;
    }
    return 0;
}

int load_programs() {
    g_modules.resize(file_count());
    for (int i = 0; i < file_count(); i++) {
        // a file of the registry that is not shipped (yet) is skipped; launching one of its kernels fails loudly
        std::string probe;
        if (!read_file(kernel_dir() + "/" + SZ_FILES[i], probe)) continue;
        if (load_file(i)) return 1;
    }
    return 0;
}

int launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz, uint32_t shared, uint64_t stream,
           const sz_arg* args, int nargs) {
    const SzEntry* e = find_entry(name);
    if (!e) return fail(std::string("no entry point ") + name + " in the registry");
    if (e->nparams != nargs) return fail(std::string(name) + " takes " + std::to_string(e->nparams) + " arguments, " + std::to_string(nargs) + " given");
    for (int i = 0; i < nargs; i++) {
        const int k = args[i].kind, p = e->kinds[i];
        const bool fits = (k == SZ_ARG_PTR && (p == SZ_P_PTR || p == SZ_P_CONSTPTR)) || (k == SZ_ARG_U32 && p == SZ_P_U32) ||
                          (k == SZ_ARG_I32 && p == SZ_P_I32) || (k == SZ_ARG_U64 && p == SZ_P_U64) || (k == SZ_ARG_F32 && p == SZ_P_F32);
        if (!fits) return fail(std::string(name) + " argument " + std::to_string(i) + ": kind " + std::to_string(k) + " does not fit parameter kind " + std::to_string(p));
    }
    if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0 || (uint64_t) bx * by * bz > 1024)
        return fail(std::string(name) + ": empty grid or a block of more than 1024 threads");
    if (ensure_init()) return 1;
    hipFunction_t fn;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        auto it = g_functions.find(name);
        if (it == g_functions.end()) {
            if (load_file(e->file)) return 1;
            hipFunction_t f = nullptr;
            if (hip_check(hip().hipModuleGetFunction(&f, g_modules[e->file].module, name), (std::string("hipModuleGetFunction(") + name + ")").c_str())) return 1;
            it = g_functions.emplace(name, f).first;
        }
        fn = it->second;
    }
    uint64_t vals[24];
    void* ptrs[24];
    for (int i = 0; i < nargs; i++) {
        vals[i] = args[i].value;   // little-endian: a 4-byte parameter reads the low half of its slot
        ptrs[i] = &vals[i];
    }
    g_launches.fetch_add(1, std::memory_order_relaxed);
    const bool timed = g_ktime && !g_capturing && std::strncmp(name, g_ktime_prefix.c_str(), g_ktime_prefix.size()) == 0;
    Timed t{e->name, nullptr, nullptr};
    if (timed && (hip_check(hip().hipEventCreate(&t.a), "hipEventCreate") || hip_check(hip().hipEventCreate(&t.b), "hipEventCreate"))) return 1;
    int r;
    if (timed && hip().hipExtModuleLaunchKernel && (uint64_t) gx * bx < (1ull << 32) && (uint64_t) gy * by < (1ull << 32) &&
        (uint64_t) gz * bz < (1ull << 32)) {
        // the two events become the dispatch's own begin and end time stamps: the kernel's duration, nothing around it
        r = hip_check(hip().hipExtModuleLaunchKernel(fn, gx * bx, gy * by, gz * bz, bx, by, bz, shared, (hipStream_t) stream, ptrs, nullptr,
                                                     t.a, t.b, 0), name);
    } else {
        if (timed && hip_check(hip().hipEventRecord(t.a, (hipStream_t) stream), "hipEventRecord")) return 1;
        r = hip_check(hip().hipModuleLaunchKernel(fn, gx, gy, gz, bx, by, bz, shared, (hipStream_t) stream, ptrs, nullptr), name);
        if (timed) hip().hipEventRecord(t.b, (hipStream_t) stream);
    }
    if (timed) {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_timed.push_back(t);
    }
    return r;
}

void set_capturing(bool on) { g_capturing += on ? 1 : -1; }

}   // namespace sz

using namespace sz;

extern "C" {

int32_t sz_device_count(int32_t* count) {
    clear_error();
    HipApi& h = hip();
    if (!h.ok) return fail(h.error);
    if (hip_check(h.hipInit(0), "hipInit")) return 1;
    int n = 0;
    if (hip_check(h.hipGetDeviceCount(&n), "hipGetDeviceCount")) return 1;
    *count = n;
    return 0;
}

int32_t sz_init(int32_t device) {
    clear_error();
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_init) return g_device == device ? 0 : fail("sz_init: already initialised on device " + std::to_string(g_device));
    HipApi& h = hip();
    if (!h.ok) return fail(h.error);
    if (hip_check(h.hipInit(0), "hipInit")) return 1;
    int n = 0;
    if (hip_check(h.hipGetDeviceCount(&n), "hipGetDeviceCount")) return 1;
    if (device < 0 || device >= n) return fail("sz_init: device " + std::to_string(device) + " of " + std::to_string(n));
    if (hip_check(h.hipSetDevice(device), "hipSetDevice")) return 1;
    if (load_programs()) return 1;
    g_device = device;
    g_init = true;
    // the static workspace's address on this device (sz_matvec_cols_static); a failure is that entry point's to report
    if (static_workspace_setup(device)) clear_error();
    return 0;
}

int32_t sz_device_name(char* buf, uint64_t len) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipDeviceGetName(buf, (int) len, g_device), "hipDeviceGetName");
}

int32_t sz_mem_info(uint64_t* free_bytes, uint64_t* total_bytes) {
    clear_error();
    if (ensure_init()) return 1;
    size_t f = 0, t = 0;
    if (hip_check(hip().hipMemGetInfo(&f, &t), "hipMemGetInfo")) return 1;
    *free_bytes = f;
    *total_bytes = t;
    return 0;
}

int32_t sz_malloc(uint64_t* dev, uint64_t bytes) {
    clear_error();
    if (ensure_init()) return 1;
    void* p = nullptr;
    if (hip_check(hip().hipMalloc(&p, bytes ? bytes : 1), "hipMalloc")) return 1;
    *dev = (uint64_t) p;
    return 0;
}
int32_t sz_free(uint64_t dev) {
    clear_error();
    if (ensure_init()) return 1;
    return dev ? hip_check(hip().hipFree((void*) dev), "hipFree") : 0;
}
int32_t sz_upload(uint64_t dev, const void* host, uint64_t bytes) {
    clear_error();
    if (ensure_init()) return 1;
    return bytes ? hip_check(hip().hipMemcpyHtoD((void*) dev, host, bytes), "hipMemcpyHtoD") : 0;
}
int32_t sz_download(void* host, uint64_t dev, uint64_t bytes) {
    clear_error();
    if (ensure_init()) return 1;
    return bytes ? hip_check(hip().hipMemcpyDtoH(host, (const void*) dev, bytes), "hipMemcpyDtoH") : 0;
}
int32_t sz_memset(uint64_t dev, int32_t byte, uint64_t bytes, uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    if (!bytes) return 0;
    // a launch of the library's own (fill_bytes, kernels/moe.hip) rather than the runtime's memset: a caller may capture it
    const uint64_t want = (bytes / 16 + 255) / 256 + 1;
    const sz_arg a[] = {P(dev), U32((uint32_t) (byte & 0xff)), U64(bytes)};
    return launch("fill_bytes", (uint32_t) std::min<uint64_t>(want, 8192), 1, 1, 256, 0, stream, a);
}
int32_t sz_stream_create(uint64_t* stream) {
    clear_error();
    if (ensure_init()) return 1;
    hipStream_t s = nullptr;
    if (hip_check(hip().hipStreamCreateWithFlags(&s, 1 /* hipStreamNonBlocking */), "hipStreamCreateWithFlags")) return 1;
    *stream = (uint64_t) s;
    return 0;
}
int32_t sz_stream_destroy(uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipStreamDestroy((hipStream_t) stream), "hipStreamDestroy");
}
int32_t sz_stream_synchronize(uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipStreamSynchronize((hipStream_t) stream), "hipStreamSynchronize");
}
int32_t sz_synchronize(void) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipDeviceSynchronize(), "hipDeviceSynchronize");
}
int32_t sz_event_create(uint64_t* event) {
    clear_error();
    if (ensure_init()) return 1;
    hipEvent_t e = nullptr;
    if (hip_check(hip().hipEventCreate(&e), "hipEventCreate")) return 1;
    *event = (uint64_t) e;
    return 0;
}
int32_t sz_event_destroy(uint64_t event) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipEventDestroy((hipEvent_t) event), "hipEventDestroy");
}
int32_t sz_event_record(uint64_t event, uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipEventRecord((hipEvent_t) event, (hipStream_t) stream), "hipEventRecord");
}
int32_t sz_stream_wait_event(uint64_t stream, uint64_t event) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipStreamWaitEvent((hipStream_t) stream, (hipEvent_t) event, 0), "hipStreamWaitEvent");
}
int32_t sz_event_synchronize(uint64_t event) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipEventSynchronize((hipEvent_t) event), "hipEventSynchronize");
}
int32_t sz_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipEventElapsedTime(ms, (hipEvent_t) start, (hipEvent_t) stop), "hipEventElapsedTime");
}
int32_t sz_capture_begin(uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    if (hip_check(hip().hipStreamBeginCapture((hipStream_t) stream, 1 /* thread-local */), "hipStreamBeginCapture")) return 1;
    set_capturing(true);
    return 0;
}
int32_t sz_capture_end(uint64_t stream, uint64_t* graph_exec) {
    clear_error();
    if (ensure_init()) return 1;
    hipGraph_t g = nullptr;
    set_capturing(false);
    if (hip_check(hip().hipStreamEndCapture((hipStream_t) stream, &g), "hipStreamEndCapture")) return 1;
    hipGraphExec_t ex = nullptr;
    const int r = hip_check(hip().hipGraphInstantiate(&ex, g, nullptr, nullptr, 0), "hipGraphInstantiate");
    hip().hipGraphDestroy(g);
    if (r) return 1;
    *graph_exec = (uint64_t) ex;
    return 0;
}
int32_t sz_graph_launch(uint64_t graph_exec, uint64_t stream) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipGraphLaunch((hipGraphExec_t) graph_exec, (hipStream_t) stream), "hipGraphLaunch");
}
int32_t sz_graph_destroy(uint64_t graph_exec) {
    clear_error();
    if (ensure_init()) return 1;
    return hip_check(hip().hipGraphExecDestroy((hipGraphExec_t) graph_exec), "hipGraphExecDestroy");
}

int32_t sz_launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz, uint32_t shared_bytes,
                  uint64_t stream, const sz_arg* args, int32_t nargs) {
    clear_error();
    return launch(name, gx, gy, gz, bx, by, bz, shared_bytes, stream, args, nargs);
}
int32_t sz_kernel_count(void) { return entry_count(); }
int32_t sz_kernel_info(int32_t i, const char** name, const char** file, int32_t* nparams, int32_t* kinds, int32_t max_params) {
    clear_error();
    const SzEntry* e = entry(i);
    if (!e) return fail("sz_kernel_info: no entry " + std::to_string(i));
    if (name) *name = e->name;
    if (file) *file = file_name(e->file);
    if (nparams) *nparams = e->nparams;
    for (int p = 0; kinds && p < e->nparams && p < max_params; p++) kinds[p] = e->kinds[p];
    return 0;
}
uint64_t sz_launch_count(void) { return g_launches.load(); }

static void ktime_clear() {
    for (auto& t : g_timed) {
        hip().hipEventDestroy(t.a);
        hip().hipEventDestroy(t.b);
    }
    g_timed.clear();
}
int32_t sz_ktime_begin(const char* prefix) {
    clear_error();
    if (ensure_init()) return 1;
    std::lock_guard<std::mutex> lock(g_mutex);
    ktime_clear();
    g_ktime_prefix = prefix ? prefix : "";
    g_ktime = true;
    return 0;
}
int32_t sz_ktime_entry(int32_t i, const char** name, uint64_t* launches, double* total_ms) {
    clear_error();
    if (ensure_init()) return 1;
    if (hip_check(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")) return 1;
    std::lock_guard<std::mutex> lock(g_mutex);
    std::vector<const char*> names;
    for (auto& t : g_timed)
        if (std::find(names.begin(), names.end(), t.name) == names.end()) names.push_back(t.name);
    if (i < 0 || i >= (int) names.size()) return fail("sz_ktime_entry: no kernel " + std::to_string(i));
    uint64_t n = 0;
    double ms = 0.0;
    for (auto& t : g_timed) {
        if (t.name != names[i]) continue;
        float one = 0.0f;
        if (hip_check(hip().hipEventElapsedTime(&one, t.a, t.b), "hipEventElapsedTime")) return 1;
        ms += one;
        n++;
    }
    *name = names[i];
    *launches = n;
    *total_ms = ms;
    return 0;
}
int32_t sz_ktime_end(void) {
    clear_error();
    if (ensure_init()) return 1;
    hip().hipDeviceSynchronize();
    std::lock_guard<std::mutex> lock(g_mutex);
    ktime_clear();
    g_ktime = false;
    return 0;
}
int32_t sz_program_cache_key(const char* file, char* hex65) {
    clear_error();
    std::string hex;
    if (cache_key(file, hex, false)) return 1;
    std::memcpy(hex65, hex.c_str(), 65);
    return 0;
}
int32_t sz_program_cache_key_rtc(const char* file, char* hex65) {
    clear_error();
    std::string hex;
    if (cache_key(file, hex, true)) return 1;
    std::memcpy(hex65, hex.c_str(), 65);
    return 0;
}
const char* sz_program_aot_options(const char* file) {
    clear_error();
    static thread_local std::string s;
    std::string src;
    if (program_source(file, src)) return nullptr;
    s = aot_options_of(src);
    return s.c_str();
}
int32_t sz_program_file_count(void) { return file_count(); }
const char* sz_program_file_name(int32_t i) { return file_name(i); }
const char* sz_cache_dir(void) {
    static thread_local std::string s;
    s = cache_dir();
    return s.c_str();
}
const char* sz_compile_options(void) { return compile_options(); }
int32_t sz_program_write_source(const char* file, const char* path) {
    clear_error();
    std::string src;
    if (program_source(file, src)) return 1;
    std::ofstream f(path, std::ios::binary);
    if (!f) return fail(std::string("cannot write ") + path);
    f.write(src.data(), (std::streamsize) src.size());
    return 0;
}
int32_t sz_rtc_compile(const char* name, const char* source, uint64_t* code_bytes, const char** log) {
    clear_error();
    static thread_local std::string s_log;
    std::vector<char> code;
    s_log.clear();
    const int r = rtc_compile(name, source, code, s_log);
    if (log) *log = s_log.c_str();
    if (code_bytes) *code_bytes = code.size();
    return r;
}

}   // extern "C"
