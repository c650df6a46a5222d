// Shared host-side helpers of libspion_hip.so: error slot, HIP status checks, handle header.
#pragma once
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

namespace spion {

// ---- process-wide error slot (read through spion_last_error) ---------------------------------
void set_error(const char* fmt, ...);
bool error_pending();

#define SPION_HIP_OK(expr)                                                                  \
    ([&]() -> bool {                                                                        \
        hipError_t _e = (expr);                                                             \
        if (_e != hipSuccess) {                                                             \
            ::spion::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),       \
                               __FILE__, __LINE__);                                         \
            return false;                                                                   \
        }                                                                                   \
        return true;                                                                        \
    }())

// Every handle starts with this header so the family-agnostic entry points can check it.
enum HandleKind : uint32_t {
    KIND_SPARSE = 0x53504e31u,  // "SPN1"
    KIND_DENSE = 0x53504e32u,   // "SPN2"
};

struct HandleHeader {
    uint32_t magic;
    hipStream_t stream;
    char err[256];  // most recent failure of a call on this handle ("" if none), besides the process-wide slot
};

// The handle the calling thread is working on (set by the handle checks of every entry point, cleared by
// entry points without a handle): set_error files the message there as well.
void note_current_handle(HandleHeader* h);

inline bool check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("launch of %s failed: %s", what, hipGetErrorString(e));
        return false;
    }
    return true;
}

// Named ranges around the phases of a call (the reference brackets its cuSPARSE steps with nvtxRangePush / Pop,
// models/block_attn.cu:163-223): with SPION_ROCTX=1 in the environment the ROCm tools library is loaded on first use
// and every PhaseRange pushes / pops a roctx range, so that a marker trace of a training step attributes host time
// per phase.  Without the switch (or the library) a PhaseRange does nothing.
struct RoctxApi {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
};
inline const RoctxApi* roctx_api() {
    static const RoctxApi api = [] {
        RoctxApi a;
        const char* env = std::getenv("SPION_ROCTX");
        if (!env || env[0] != '1') return a;
        void* h = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
        if (!h) h = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
        if (!h) return a;
        a.push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
        a.pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
        if (!a.push || !a.pop) a = RoctxApi{};
        return a;
    }();
    return api.push ? &api : nullptr;
}
struct PhaseRange {
    const RoctxApi* api;
    explicit PhaseRange(const char* name) : api(roctx_api()) {
        if (api) api->push(name);
    }
    ~PhaseRange() {
        if (api) api->pop();
    }
    PhaseRange(const PhaseRange&) = delete;
    PhaseRange& operator=(const PhaseRange&) = delete;
};

}  // namespace spion
