// Device/runtime plumbing of the C ABI: init, memory, copies, events, error string.
#include "runtime.hpp"
#include "../../include/powerinfer_hip.h"

#include <stdio.h>
#include <string.h>

namespace pi {

static thread_local char g_err[512] = "";

void set_error(const char * msg) { snprintf(g_err, sizeof g_err, "%s", msg); }
int fail(int code, const char * msg) { set_error(msg); return code; }
int hip_fail(hipError_t e, const char * what) {
    snprintf(g_err, sizeof g_err, "%s: %s", what, hipGetErrorString(e));
    return PI_E_HIP;
}
int check_launch(const char * what) {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? PI_OK : hip_fail(e, what);
}

}  // namespace pi

namespace pi {
int compute_units() {
    static int cached[16] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 0;
    if (!cached[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev] = n;
    }
    return cached[dev];
}
}  // namespace pi

extern "C" {

const char * pi_last_error(void) { return pi::g_err; }

int pi_init(int device) {
    int n = 0;
    PI_HIP_TRY(hipGetDeviceCount(&n));
    if (n <= 0) return pi::fail(PI_E_HIP, "pi_init: no HIP device; this library has no CPU fallback");
    if (device < 0 || device >= n) return pi::fail(PI_E_ARG, "pi_init: device index out of range");
    PI_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t p;
    PI_HIP_TRY(hipGetDeviceProperties(&p, device));
    if (p.warpSize != 64) return pi::fail(PI_E_UNSUPPORTED, "pi_init: kernels are written for 64-wide wavefronts");
    (void)pi::compute_units();
    return pi::noalloc_setup();
}

int pi_device_name(char * buf, size_t n) {
    int dev = 0;
    PI_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t p;
    PI_HIP_TRY(hipGetDeviceProperties(&p, dev));
    snprintf(buf, n, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
    return PI_OK;
}

void * pi_malloc(size_t bytes) {
    void * p = nullptr;
    const hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) { pi::hip_fail(e, "hipMalloc"); return nullptr; }
    return p;
}
int pi_free(void * dptr) { if (dptr) PI_HIP_TRY(hipFree(dptr)); return PI_OK; }
void * pi_malloc_host(size_t bytes) {
    void * p = nullptr;
    const hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocCoherent);
    if (e != hipSuccess) { pi::hip_fail(e, "hipHostMalloc"); return nullptr; }
    return p;
}
int pi_free_host(void * hptr) { if (hptr) PI_HIP_TRY(hipHostFree(hptr)); return PI_OK; }
int pi_memset(void * dptr, int byte, size_t bytes) { PI_HIP_TRY(hipMemset(dptr, byte, bytes)); return PI_OK; }
int pi_memcpy_h2d(void * dptr, const void * host, size_t bytes) { PI_HIP_TRY(hipMemcpy(dptr, host, bytes, hipMemcpyHostToDevice)); return PI_OK; }
int pi_memcpy_d2h(void * host, const void * dptr, size_t bytes) { PI_HIP_TRY(hipMemcpy(host, dptr, bytes, hipMemcpyDeviceToHost)); return PI_OK; }
int pi_memcpy_d2d(void * dst, const void * src, size_t bytes) { PI_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice)); return PI_OK; }
int pi_sync(void) { PI_HIP_TRY(hipDeviceSynchronize()); return PI_OK; }

void * pi_event_create(void) {
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) { pi::set_error("hipEventCreate failed"); return nullptr; }
    return (void *)e;
}
int pi_event_record(void * ev, pi_stream_t stream) { PI_HIP_TRY(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream)); return PI_OK; }
int pi_event_elapsed_ms(void * start, void * stop, float * ms) {
    PI_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
    PI_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return PI_OK;
}
int pi_event_destroy(void * ev) { PI_HIP_TRY(hipEventDestroy((hipEvent_t)ev)); return PI_OK; }

}  // extern "C"
