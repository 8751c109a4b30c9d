// Error plumbing shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/verinf_hip.h"

namespace vi {

inline char *err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline bool is_pow2(long long x) { return x > 0 && (x & (x - 1)) == 0; }
inline int ilog2(long long x) {
    int l = 0;
    while ((1ll << l) < x) ++l;
    return l;
}

}  // namespace vi

#define VI_HIP(call)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) return vi::fail(VI_EHIP, "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)

#define VI_LAUNCH_CHECK(name)                                                             \
    do {                                                                                  \
        hipError_t e_ = hipGetLastError();                                                \
        if (e_ != hipSuccess) return vi::fail(VI_EHIP, "launch %s: %s", name, hipGetErrorString(e_)); \
    } while (0)
