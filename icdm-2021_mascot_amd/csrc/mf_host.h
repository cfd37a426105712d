// Host-side helpers shared by the extern "C" translation units: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "../../include/mascot_hip.h"

namespace mf {

void set_error(const char* fmt, ...);

inline int check_hip(hipError_t e, const char* what)
{
    if (e == hipSuccess) return MF_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return (int)e;
}
inline int launch_status(const char* what) { return check_hip(hipGetLastError(), what); }
inline int invalid(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
inline int invalid(const char* fmt, ...)
{
    char buf[256];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    set_error("%s", buf);
    return MF_EINVAL;
}
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace mf
