// Run-time binding of libamdhip64 and libhiprtc: dlopen + dlsym of exactly the entry points the hot path needs, the
// counterpart of crates/shadowzero-cuda/src/{dylib,driver,nvrtc}.rs.  A missing library is an error value, not a crash
// (driver.rs:200-222): callers on a machine without ROCm get a clean "not available".
#include <dlfcn.h>

#include <cstdlib>
#include <cstring>
#include <mutex>

#include "sz_internal.hpp"

namespace sz {

static thread_local std::string g_error;

int fail(const std::string& msg) {
    g_error = msg;
    return 1;
}
void clear_error() { g_error.clear(); }
const char* last_error_cstr() { return g_error.c_str(); }

static void* open_first(const char* env, std::initializer_list<const char*> names, std::string& tried) {
    if (const char* e = std::getenv(env)) {
        if (void* h = dlopen(e, RTLD_NOW | RTLD_GLOBAL)) return h;
        tried += std::string(e) + " (" + dlerror() + "); ";
    }
    for (const char* n : names) {
        if (void* h = dlopen(n, RTLD_NOW | RTLD_GLOBAL)) return h;
        tried += std::string(n) + "; ";
    }
    return nullptr;
}

template <class F>
static bool bind(void* lib, const char* name, F& fn, std::string& missing) {
    fn = reinterpret_cast<F>(dlsym(lib, name));
    if (!fn) missing += std::string(name) + " ";
    return fn != nullptr;
}

static void* g_hip_lib = nullptr;   // the bound libamdhip64, for the registration forwarders below

HipApi& hip() {
    static HipApi api;
    static std::once_flag once;
    std::call_once(once, [] {
        std::string tried;
        // never unloaded, like the reference's libraries (dylib.rs:19-20)
        void* lib = g_hip_lib = open_first("SHADOWZERO_HIP_LIB", {"libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6", "/opt/rocm/lib/libamdhip64.so"}, tried);
        if (!lib) {
            api.error = "libamdhip64 not found (tried " + tried + ")";
            return;
        }
        std::string missing;
#define SZ_BIND(f) bind(lib, #f, api.f, missing)
        SZ_BIND(hipInit);
        SZ_BIND(hipGetDeviceCount);
        SZ_BIND(hipSetDevice);
        SZ_BIND(hipDeviceGetName);
        SZ_BIND(hipMemGetInfo);
        SZ_BIND(hipMalloc);
        SZ_BIND(hipFree);
        SZ_BIND(hipHostMalloc);
        SZ_BIND(hipHostFree);
        SZ_BIND(hipMemcpyHtoD);
        SZ_BIND(hipMemcpyDtoH);
        SZ_BIND(hipMemcpyDtoHAsync);
        SZ_BIND(hipMemcpyHtoDAsync);
        SZ_BIND(hipMemsetD8Async);
        SZ_BIND(hipModuleLoadData);
        SZ_BIND(hipModuleUnload);
        SZ_BIND(hipModuleGetFunction);
        SZ_BIND(hipModuleLaunchKernel);
        {
            std::string optional;   // absent from an old runtime: timed launches then fall back to events either side
            bind(lib, "hipExtModuleLaunchKernel", api.hipExtModuleLaunchKernel, optional);
        }
        SZ_BIND(hipStreamCreateWithFlags);
        SZ_BIND(hipStreamDestroy);
        SZ_BIND(hipStreamSynchronize);
        SZ_BIND(hipDeviceSynchronize);
        SZ_BIND(hipEventCreate);
        SZ_BIND(hipEventDestroy);
        SZ_BIND(hipEventRecord);
        SZ_BIND(hipEventSynchronize);
        SZ_BIND(hipStreamWaitEvent);
        SZ_BIND(hipEventElapsedTime);
        SZ_BIND(hipStreamBeginCapture);
        SZ_BIND(hipStreamEndCapture);
        SZ_BIND(hipGraphInstantiate);
        SZ_BIND(hipGraphLaunch);
        SZ_BIND(hipGraphExecDestroy);
        SZ_BIND(hipGraphDestroy);
        SZ_BIND(hipGetErrorName);
        SZ_BIND(hipGetErrorString);
#undef SZ_BIND
        if (!missing.empty()) {
            api.error = "libamdhip64 lacks: " + missing;
            return;
        }
        api.ok = true;
    });
    return api;
}

void* hip_symbol(const char* name) {
    hip();
    return g_hip_lib ? dlsym(g_hip_lib, name) : nullptr;
}

int hip_check(hipError_t e, const char* call) {
    if (e == 0) return 0;
    HipApi& h = hip();
    std::string name = h.ok ? h.hipGetErrorName(e) : "?", text = h.ok ? h.hipGetErrorString(e) : "?";
    return fail(std::string(call) + ": " + name + " (" + text + ", code " + std::to_string(e) + ")");
}

RtcApi& rtc() {
    static RtcApi api;
    static std::once_flag once;
    std::call_once(once, [] {
        std::string tried;
        void* lib = open_first("SHADOWZERO_HIPRTC_LIB", {"libhiprtc.so", "libhiprtc.so.7", "libhiprtc.so.6", "/opt/rocm/lib/libhiprtc.so"}, tried);
        if (!lib) {
            api.error = "libhiprtc not found (tried " + tried + ")";
            return;
        }
        std::string missing;
#define SZ_BIND(f) bind(lib, #f, api.f, missing)
        SZ_BIND(hiprtcCreateProgram);
        SZ_BIND(hiprtcCompileProgram);
        SZ_BIND(hiprtcGetProgramLogSize);
        SZ_BIND(hiprtcGetProgramLog);
        SZ_BIND(hiprtcGetCodeSize);
        SZ_BIND(hiprtcGetCode);
        SZ_BIND(hiprtcDestroyProgram);
        SZ_BIND(hiprtcGetErrorString);
#undef SZ_BIND
        if (!missing.empty()) {
            api.error = "libhiprtc lacks: " + missing;
            return;
        }
        api.ok = true;
    });
    return api;
}

int rtc_compile(const char* name, const std::string& source, std::vector<char>& code, std::string& log) {
    RtcApi& r = rtc();
    if (!r.ok) return fail(r.error);
    void* prog = nullptr;
    int e = r.hiprtcCreateProgram(&prog, source.c_str(), name, 0, nullptr, nullptr);
    if (e) return fail(std::string("hiprtcCreateProgram: ") + r.hiprtcGetErrorString(e));
    // the options of compile_options(), one token each, plus the target
    std::vector<std::string> opts{"--offload-arch=gfx950"};
    {
        std::string all = compile_options(), tok;
        for (size_t i = 0; i <= all.size(); i++) {
            if (i == all.size() || all[i] == ' ') {
                if (!tok.empty()) opts.push_back(tok);
                tok.clear();
            } else {
                tok += all[i];
            }
        }
    }
    std::vector<const char*> optv;
    for (auto& o : opts) optv.push_back(o.c_str());
    e = r.hiprtcCompileProgram(prog, (int) optv.size(), optv.data());
    size_t n = 0;
    if (r.hiprtcGetProgramLogSize(prog, &n) == 0 && n > 1) {
        log.resize(n);
        r.hiprtcGetProgramLog(prog, log.data());
    }
    if (e) {
        r.hiprtcDestroyProgram(&prog);
        return fail(std::string("hiprtcCompileProgram(") + name + "): " + r.hiprtcGetErrorString(e) + "\n" + log);   // the full log, nvrtc.rs:225-227
    }
    size_t cn = 0;
    e = r.hiprtcGetCodeSize(prog, &cn);
    if (!e) {
        code.resize(cn);
        e = r.hiprtcGetCode(prog, code.data());
    }
    r.hiprtcDestroyProgram(&prog);
    if (e) return fail(std::string("hiprtcGetCode: ") + r.hiprtcGetErrorString(e));
    return 0;
}

}   // namespace sz

extern "C" const char* sz_last_error(void) { return sz::last_error_cstr(); }

// ---- what a hipcc-compiled translation unit of this library (csrc/static_workspace.hip: a `static __device__` array and
// the host code that asks for its address) expects from the HIP runtime it would normally be linked against: the
// registration of its device code at load time and two runtime calls.  They are forwarded to the library bound above, so
// this library still links no ROCm library and there is one HIP runtime in the process; without libamdhip64 they do
// nothing and the entry point that needs them reports it.  Hidden: nothing outside this library binds to them.
extern "C" {
#define SZ_HIDDEN __attribute__((visibility("hidden")))
SZ_HIDDEN void** __hipRegisterFatBinary(const void* data) {
    auto f = reinterpret_cast<void** (*)(const void*)>(sz::hip_symbol("__hipRegisterFatBinary"));
    return f ? f(data) : nullptr;
}
SZ_HIDDEN void __hipRegisterVar(void** modules, void* var, char* host_name, char* device_name, int ext, size_t size, int constant, int global) {
    auto f = reinterpret_cast<void (*)(void**, void*, char*, char*, int, size_t, int, int)>(sz::hip_symbol("__hipRegisterVar"));
    if (f && modules) f(modules, var, host_name, device_name, ext, size, constant, global);
}
SZ_HIDDEN void __hipUnregisterFatBinary(void** modules) {
    auto f = reinterpret_cast<void (*)(void**)>(sz::hip_symbol("__hipUnregisterFatBinary"));
    if (f && modules) f(modules);
}
SZ_HIDDEN int hipGetSymbolAddress(void** dev_ptr, const void* symbol) {
    auto f = reinterpret_cast<int (*)(void**, const void*)>(sz::hip_symbol("hipGetSymbolAddress"));
    return f ? f(dev_ptr, symbol) : 1;   // hipErrorInvalidValue
}
SZ_HIDDEN int hipGetDevice(int* device) {
    auto f = reinterpret_cast<int (*)(int*)>(sz::hip_symbol("hipGetDevice"));
    return f ? f(device) : 1;
}
#undef SZ_HIDDEN
}
