// sz_matvec_cols_static: sz_matvec_cols for callers that cannot allocate device memory or hand over a workspace (code
// under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The EXL3 kernels' workspace (the one-matrix
// plan and the split-k partial sums, sz_matvec_cols_scratch() bytes) lives in a device array of this library instead.
//
// This is the one file of the library that hipcc compiles as host + device code: the array is a `static __device__`
// object of this file, and its device address on a GPU is only known to the HIP runtime, which hands it out through
// hipGetSymbolAddress.  In host code the array's name stands for a host-side shadow object, never for device memory, so the
// host code below uses the looked-up address `g_workspace[device]` everywhere and the name `scratch` only inside
// HIP_SYMBOL().  The kernels are the ones sz_matvec_cols launches; they take the address as an argument.
//
// The registration calls hipcc emits for this file and the two runtime calls below resolve to forwarders inside the
// library (csrc/hipbind.cpp) that pass them to the libamdhip64 bound at run time.
#include <hip/hip_runtime.h>

#include <atomic>
#include <string>

#include "shadowzero_hip.h"

namespace sz {
int fail(const std::string& msg);
void clear_error();
int ensure_init();
int matvec_cols_dev(int ty, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys, uint32_t m, uint64_t scratch,
                    uint64_t scratch_bytes, uint64_t stream);
int static_workspace_setup(int device);
}   // namespace sz

// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.
static __device__ __align__(256) unsigned char scratch[SZ_STATIC_WORKSPACE_BYTES];

enum { SZ_MAX_DEVICES = 64 };
// the array's device address on each GPU that has been set up; sz_init and the entry point may look it up from different
// host threads at the same time (both find the same address), hence atomic
static std::atomic<void*> g_workspace[SZ_MAX_DEVICES];

// Called by sz_init with `device` current (and by the entry point for a device it has not seen).
int sz::static_workspace_setup(int device) {
    if (device < 0 || device >= SZ_MAX_DEVICES) return fail("static workspace: device " + std::to_string(device) + " is out of range");
    if (g_workspace[device].load(std::memory_order_acquire)) return 0;
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
        return fail("hipGetSymbolAddress(static workspace) on device " + std::to_string(device) + ": code " + std::to_string((int) e));
    g_workspace[device].store(ptr, std::memory_order_release);
    return 0;
}

extern "C" int32_t sz_matvec_cols_static(int32_t ggml_type, uint64_t w, uint64_t cols, uint64_t rows, uint64_t x, uint32_t xs, uint64_t y, uint32_t ys,
                                         uint32_t m, uint64_t stream) {
    sz::clear_error();
    if (sz::ensure_init()) return 1;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) return sz::fail("sz_matvec_cols_static: hipGetDevice failed");
    if (sz::static_workspace_setup(device)) return 1;
    // the size check comes before any launch: a product whose plan and partial sums do not fit the array is refused
    const uint64_t need = sz_matvec_cols_scratch(ggml_type, cols, rows, m);
    if (need > SZ_STATIC_WORKSPACE_BYTES)
        return sz::fail("sz_matvec_cols_static: this product needs " + std::to_string(need) + " bytes of workspace, the static one holds " +
                        std::to_string((uint64_t) SZ_STATIC_WORKSPACE_BYTES) + "; use sz_matvec_cols with a workspace of the caller's");
    // nothing in the workspace has to start at zero: the plan launch writes every table entry it reads and the partial sums
    // are all written before the finishing launch adds them, so the last call's contents are simply overwritten
    return sz::matvec_cols_dev(ggml_type, w, cols, rows, x, xs, y, ys, m, (uint64_t) g_workspace[device].load(std::memory_order_acquire), SZ_STATIC_WORKSPACE_BYTES, stream);
}
