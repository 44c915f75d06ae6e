// The HIP runtime, reached through dlopen/dlsym like the reference reaches its
// drivers (jit/gpu/hip/hipapi.go:43-114): no link-time dependency, and a
// process that already holds a HIP runtime (for instance one bundled with a
// Python framework) keeps exactly one -- two runtimes in one process cannot
// both open the device.
#pragma once
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <string>

struct HipApi {
    void* handle = nullptr;
    std::string path;

    hipError_t (*SetDevice)(int) = nullptr;
    hipError_t (*GetDeviceProperties)(hipDeviceProp_t*, int) = nullptr;
    const char* (*GetErrorString)(hipError_t) = nullptr;
    hipError_t (*StreamCreate)(hipStream_t*) = nullptr;
    hipError_t (*StreamDestroy)(hipStream_t) = nullptr;
    hipError_t (*StreamSynchronize)(hipStream_t) = nullptr;
    hipError_t (*DeviceSynchronize)() = nullptr;
    hipError_t (*ModuleLoad)(hipModule_t*, const char*) = nullptr;
    hipError_t (*ModuleUnload)(hipModule_t) = nullptr;
    hipError_t (*ModuleGetFunction)(hipFunction_t*, hipModule_t, const char*) = nullptr;
    hipError_t (*ModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned,
                                     unsigned, unsigned, hipStream_t, void**, void**) = nullptr;
    hipError_t (*Malloc)(void**, size_t) = nullptr;
    hipError_t (*Free)(void*) = nullptr;
    hipError_t (*Memcpy)(void*, const void*, size_t, hipMemcpyKind) = nullptr;
    hipError_t (*MemcpyAsync)(void*, const void*, size_t, hipMemcpyKind, hipStream_t) = nullptr;
    hipError_t (*GetLastError)() = nullptr;
};

// Resolves the runtime once.  Returns null (and sets *why) when no HIP runtime
// can be loaded or a symbol is missing.
inline const HipApi* hip_api(std::string* why) {
    static HipApi api;
    static bool tried = false, ok = false;
    static std::string err;
    if (!tried) {
        tried = true;
        const char* names[] = {"libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6"};
        for (const char* n : names)  // a runtime this process already holds
            if ((api.handle = dlopen(n, RTLD_NOW | RTLD_NOLOAD))) { api.path = n; break; }
        if (!api.handle) {
            const char* files[] = {"/opt/rocm/lib/libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so"};
            for (const char* n : files)
                if ((api.handle = dlopen(n, RTLD_NOW | RTLD_GLOBAL))) { api.path = n; break; }
        }
        if (!api.handle) {
            err = std::string("cannot load the HIP runtime: ") + dlerror();
        } else {
            ok = true;
            auto sym = [&](const char* n, const char* alt = nullptr) -> void* {
                void* p = dlsym(api.handle, n);
                if (!p && alt) p = dlsym(api.handle, alt);
                if (!p && ok) { ok = false; err = std::string("HIP runtime lacks ") + n; }
                return p;
            };
#define JL_SYM(field, name, ...) api.field = (decltype(api.field))sym(name, ##__VA_ARGS__)
            JL_SYM(SetDevice, "hipSetDevice");
            // the properties call is versioned by struct layout; the headers here are the R0600 layout
            JL_SYM(GetDeviceProperties, "hipGetDevicePropertiesR0600", "hipGetDeviceProperties");
            JL_SYM(GetErrorString, "hipGetErrorString");
            JL_SYM(StreamCreate, "hipStreamCreate");
            JL_SYM(StreamDestroy, "hipStreamDestroy");
            JL_SYM(StreamSynchronize, "hipStreamSynchronize");
            JL_SYM(DeviceSynchronize, "hipDeviceSynchronize");
            JL_SYM(ModuleLoad, "hipModuleLoad");
            JL_SYM(ModuleUnload, "hipModuleUnload");
            JL_SYM(ModuleGetFunction, "hipModuleGetFunction");
            JL_SYM(ModuleLaunchKernel, "hipModuleLaunchKernel");
            JL_SYM(Malloc, "hipMalloc");
            JL_SYM(Free, "hipFree");
            JL_SYM(Memcpy, "hipMemcpy");
            JL_SYM(MemcpyAsync, "hipMemcpyAsync");
            JL_SYM(GetLastError, "hipGetLastError");
#undef JL_SYM
        }
    }
    if (!ok) {
        if (why) *why = err;
        return nullptr;
    }
    return &api;
}
