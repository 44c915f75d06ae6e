// The one workspace of the library that is not allocated: a file-scope device array that
// every GPU the library runs on holds from the moment the library is loaded until the process
// ends.  It serves jl_matmul_static_dev, the entry point for callers that cannot allocate
// (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc).
//
// In host code the array's NAME is only a stand-in for the device variable, not a device
// address: passing it to a kernel compiles and then faults on the GPU.  The address a kernel
// may use is what hipGetSymbolAddress returns, and each GPU holds its own copy of the array at
// its own address, so it is looked up once per device, with that device current, and kept.
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "scratch.h"

static __device__ __align__(256) unsigned char scratch[JL_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_mu;
void* g_ptr[kMaxDevices];          // per device: the array's address on that device
bool g_tried[kMaxDevices];
std::string g_err[kMaxDevices];
}  // namespace

// The device address of `scratch` on `device`, which must be the calling thread's current
// device (jl_ctx_create calls this right after hipSetDevice).  Returns 0 and the address, or
// the HIP error code with *err set to its text.
extern "C" __attribute__((visibility("hidden"))) int jl_static_scratch_get(int device, void** ptr, size_t* bytes,
                                                                          const char** err) {
    *ptr = nullptr;
    *bytes = 0;
    if (device < 0 || device >= kMaxDevices) {
        *err = "device ordinal outside the static scratch table";
        return (int)hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_tried[device]) {
        g_tried[device] = true;
        int cur = -1;
        hipError_t e = hipGetDevice(&cur);
        if (e == hipSuccess && cur != device) e = hipErrorInvalidDevice;   // the lookup answers for the current device
        void* p = nullptr;
        if (e == hipSuccess) e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            g_err[device] = std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e);
            g_ptr[device] = nullptr;
        } else {
            g_ptr[device] = p;
        }
    }
    if (!g_ptr[device]) {
        *err = g_err[device].c_str();
        return (int)hipErrorInvalidSymbol;
    }
    *ptr = g_ptr[device];
    *bytes = JL_STATIC_SCRATCH_BYTES;
    return 0;
}
