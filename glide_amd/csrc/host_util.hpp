// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/glide_hip.h"

#define GLIDE_HIP_TRY(expr)                                  \
    do {                                                     \
        hipError_t _e = (expr);                              \
        if (_e != hipSuccess) return static_cast<int>(_e);   \
    } while (0)

namespace glide {
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? GLIDE_OK : static_cast<int>(e);
}
}  // namespace glide
