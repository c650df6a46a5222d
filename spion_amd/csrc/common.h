// Shared host-side helpers of libspion_hip.so: error slot, HIP status checks, handle header.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
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

}  // namespace spion
