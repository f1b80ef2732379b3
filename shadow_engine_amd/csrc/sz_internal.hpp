// Internal declarations of libshadowzero_hip: the run-time HIP binding, the kernel programs and the launch helper.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "shadowzero_hip.h"

namespace sz {

// ---- error reporting --------------------------------------------------------------------------------------------
int fail(const std::string& msg);            // records msg for sz_last_error, returns 1
void clear_error();

// ---- the HIP driver/runtime entry points this library uses, bound by hand with dlsym (no ROCm header is included):
// the 1:1 replacement of the cu* table of crates/shadowzero-cuda/src/driver.rs:132-196.
typedef int hipError_t;
typedef void* hipStream_t;
typedef void* hipEvent_t;
typedef void* hipModule_t;
typedef void* hipFunction_t;
typedef void* hipGraph_t;
typedef void* hipGraphExec_t;

struct HipApi {
    bool ok = false;
    std::string error;
    hipError_t (*hipInit)(unsigned);
    hipError_t (*hipGetDeviceCount)(int*);
    hipError_t (*hipSetDevice)(int);
    hipError_t (*hipDeviceGetName)(char*, int, int);
    hipError_t (*hipMemGetInfo)(size_t*, size_t*);
    hipError_t (*hipMalloc)(void**, size_t);
    hipError_t (*hipFree)(void*);
    hipError_t (*hipHostMalloc)(void**, size_t, unsigned);   // pinned staging buffers of the checkpoint loaders
    hipError_t (*hipHostFree)(void*);
    hipError_t (*hipMemcpyHtoD)(void*, const void*, size_t);
    hipError_t (*hipMemcpyDtoH)(void*, const void*, size_t);
    hipError_t (*hipMemcpyDtoHAsync)(void*, const void*, size_t, hipStream_t);
    hipError_t (*hipMemcpyHtoDAsync)(void*, const void*, size_t, hipStream_t);
    hipError_t (*hipMemsetD8Async)(void*, unsigned char, size_t, hipStream_t);
    hipError_t (*hipModuleLoadData)(hipModule_t*, const void*);
    hipError_t (*hipModuleUnload)(hipModule_t);
    hipError_t (*hipModuleGetFunction)(hipFunction_t*, hipModule_t, const char*);
    hipError_t (*hipModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned, hipStream_t,
                                        void**, void**);
    // optional: the launch whose start and stop events are the dispatch's own begin and end time stamps (global size in threads)
    hipError_t (*hipExtModuleLaunchKernel)(hipFunction_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, size_t, hipStream_t,
                                           void**, void**, hipEvent_t, hipEvent_t, uint32_t);
    hipError_t (*hipStreamCreateWithFlags)(hipStream_t*, unsigned);
    hipError_t (*hipStreamDestroy)(hipStream_t);
    hipError_t (*hipStreamSynchronize)(hipStream_t);
    hipError_t (*hipDeviceSynchronize)();
    hipError_t (*hipEventCreate)(hipEvent_t*);
    hipError_t (*hipEventDestroy)(hipEvent_t);
    hipError_t (*hipEventRecord)(hipEvent_t, hipStream_t);
    hipError_t (*hipEventSynchronize)(hipEvent_t);
    hipError_t (*hipStreamWaitEvent)(hipStream_t, hipEvent_t, unsigned int);
    hipError_t (*hipEventElapsedTime)(float*, hipEvent_t, hipEvent_t);
    hipError_t (*hipStreamBeginCapture)(hipStream_t, int);
    hipError_t (*hipStreamEndCapture)(hipStream_t, hipGraph_t*);
    hipError_t (*hipGraphInstantiate)(hipGraphExec_t*, hipGraph_t, void*, char*, size_t);
    hipError_t (*hipGraphLaunch)(hipGraphExec_t, hipStream_t);
    hipError_t (*hipGraphExecDestroy)(hipGraphExec_t);
    hipError_t (*hipGraphDestroy)(hipGraph_t);
    const char* (*hipGetErrorName)(hipError_t);
    const char* (*hipGetErrorString)(hipError_t);
};
HipApi& hip();                                  // binds on first use; hip().ok says whether it worked
int hip_check(hipError_t e, const char* call);  // 0, or fail("call: name (string)")
void* hip_symbol(const char* name);             // any other entry point of the bound libamdhip64 (nullptr: not there)

// hiprtc, bound the same way (the nvrtc* table of crates/shadowzero-cuda/src/nvrtc.rs:21-37); optional.
struct RtcApi {
    bool ok = false;
    std::string error;
    int (*hiprtcCreateProgram)(void**, const char*, const char*, int, const char**, const char**);
    int (*hiprtcCompileProgram)(void*, int, const char**);
    int (*hiprtcGetProgramLogSize)(void*, size_t*);
    int (*hiprtcGetProgramLog)(void*, char*);
    int (*hiprtcGetCodeSize)(void*, size_t*);
    int (*hiprtcGetCode)(void*, char*);
    int (*hiprtcDestroyProgram)(void**);
    const char* (*hiprtcGetErrorString)(int);
};
RtcApi& rtc();
// Compiles `source` for gfx950 with the library's options; fills code (the code object) and log.  0 = ok.
int rtc_compile(const char* name, const std::string& source, std::vector<char>& code, std::string& log);

// ---- kernel programs --------------------------------------------------------------------------------------------
struct SzEntry {
    const char* name;
    int file;
    int nparams;
    int kinds[24];
};
int entry_count();
const SzEntry* entry(int i);
const SzEntry* find_entry(const char* name);
int file_count();
const char* file_name(int i);
std::string kernel_dir();
std::string cache_dir();
const char* compile_options();
int program_source(const char* file, std::string& out);   // prelude + headers + file
int cache_key(const char* file, std::string& hex, bool run_time);   // of the object hipcc builds ahead of time, or of the one hiprtc builds
std::string aot_options_of(const std::string& assembled_source);    // compile_options() + the file's `// hipcc:` lines
std::string sha256_hex(const std::string& data);

bool initialized();
int ensure_init();          // fail() unless sz_init succeeded
int load_programs();        // every kernel file: cache hit or hiprtc compile, then hipModuleLoadData

// The checked launch (kernels.rs:546-598).
int launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz, uint32_t shared, uint64_t stream,
           const sz_arg* args, int nargs);

inline sz_arg P(uint64_t p) { return sz_arg{SZ_ARG_PTR, 0, p}; }
inline sz_arg U32(uint32_t v) { return sz_arg{SZ_ARG_U32, 0, v}; }
inline sz_arg U64(uint64_t v) { return sz_arg{SZ_ARG_U64, 0, v}; }
inline sz_arg F32(float v) {
    uint32_t b;
    std::memcpy(&b, &v, 4);
    return sz_arg{SZ_ARG_F32, 0, b};   // the value's bits in the low word, as sz_launch's callers pass it
}

template <size_t N>
int launch(const char* name, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t shared, uint64_t stream, const sz_arg (&args)[N]) {
    return launch(name, gx, gy, gz, bx, 1, 1, shared, stream, args, (int) N);
}

// ---- formats ------------------------------------------------------------------------------------------------------
struct Format {
    bool exl3 = false;
    bool dense = false;      // F32 / F16 / BF16: no blocks (qk = 1, bb = bytes a weight)
    int bits = 0;            // EXL3 K
    bool half = false;       // EXL3 K + 1/2 bits a weight
    uint32_t qk = 0, bb = 0; // GGUF block: weights, bytes
    const char* tag = "";    // kernel name suffix: "q8_0", "iq3_s", "exl3_3"
};
bool format_of(int ggml_type, Format& f, std::string& tag_storage);
uint64_t matrix_bytes(const Format& f, uint64_t cols, uint64_t rows);
uint32_t rows_per_block(const Format& f, uint32_t cols, uint32_t cap = 64, uint32_t lds = 16384);   // rpb of the staged GGUF kernels (0: shape not supported by them)
uint32_t exl3_ksplit(uint32_t in_f);
// y_j = W x_j, j < m <= 8, on device addresses (sz_matvec_cols): launches only, nothing is allocated.
int matvec_cols_dev(int ty, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys, uint32_t m, uint64_t scratch,
                    uint64_t scratch_bytes, uint64_t stream);
// The library's static device workspace (csrc/static_workspace.hip): its address on `device`, which must be current, is
// looked up once and kept.  0 = ok.
int static_workspace_setup(int device);

}   // namespace sz
