// Host-side helpers shared by the entry points: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/pam_hip.h"

namespace pamhost {

inline char* error_buffer()
{
    static thread_local char buf[512] = "";
    return buf;
}

inline int fail(int code, const char* fmt, ...)
{
    va_list ap; va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PAM_HIP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return PAM_HIP_OK;
}

}  // namespace pamhost
