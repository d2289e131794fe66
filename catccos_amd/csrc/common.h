// Shared plumbing of the HIP library: error reporting and argument checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "catccos_hip.h"

namespace cch {

// Records a message for cch_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Empties the calling thread's message (a call that succeeds without a note leaves none behind).
void clear_error();

#define CCH_HIP(call)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return ::cch::fail(CCH_EHIP, "%s:%d %s -> %s", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
    } while (0)

#define CCH_REQUIRE(cond, ...)                                  \
    do {                                                        \
        if (!(cond)) return ::cch::fail(CCH_EINVAL, __VA_ARGS__); \
    } while (0)

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Checks the launch that was just enqueued.
inline int launch_status(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(CCH_EHIP, "launch of %s failed: %s", what, hipGetErrorString(e));
    return CCH_OK;
}

}  // namespace cch
