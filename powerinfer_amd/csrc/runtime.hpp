// Host-side runtime plumbing shared by the launchers: error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>

namespace pi {

void set_error(const char * msg);
int  fail(int code, const char * msg);                 // records msg, returns code
int  hip_fail(hipError_t e, const char * what);        // records "what: hipGetErrorString", returns PI_E_HIP
int  check_launch(const char * what);                  // hipGetLastError() after a kernel launch
int  compute_units();                                  // compute units of the current device (0 on error); cached per device, allocates nothing
int  noalloc_setup();                                  // resolves the static scratch array of pi_k_sparse_ffn_noalloc on the current device

}  // namespace pi

#define PI_HIP_TRY(expr)                                          \
    do {                                                          \
        hipError_t _e = (expr);                                   \
        if (_e != hipSuccess) return pi::hip_fail(_e, #expr);     \
    } while (0)
