// Error reporting and version of the C ABI.
#include "akv_common.h"

#include <stdarg.h>

namespace akv {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return AKV_ERR_LAUNCH;
    }
    return AKV_OK;
}

int g_tune_epoch = 0;

int compute_units() {
    // per device: a process may use several
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
        cached[dev] = n > 0 ? n : -1;
    }
    return cached[dev] > 0 ? cached[dev] : 0;
}

}  // namespace akv

extern "C" int akv_reload_tuning(void) {
    ++akv::g_tune_epoch;
    return AKV_OK;
}

// Plain streaming copy, 16 bytes per thread and iteration: the known-size kernel that hardware byte
// counters of the other kernels are scaled against.
__global__ __launch_bounds__(256) void copy_probe_kernel(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

extern "C" int akv_copy_probe(void *dst, const void *src, size_t bytes, akv_stream_t stream) {
    AKV_REQUIRE(dst && src && bytes % 16 == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0,
                "copy_probe: needs 16-byte aligned pointers and size");
    hipLaunchKernelGGL(copy_probe_kernel, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<u32x4 *>(dst), static_cast<const u32x4 *>(src), bytes / 16);
    return akv::check_launch("copy_probe");
}

extern "C" int akv_version(void) { return 100; }

extern "C" const char *akv_last_error(void) { return akv::g_error; }
