// Library-level entry points: version, status names, device check.
#include "common.h"
#include <string.h>

extern "C" int trn_version(void) { return 100; }  // 0.1.0

extern "C" const char* trn_status_name(int status) {
    switch (status) {
        case TRN_OK: return "TRN_OK";
        case TRN_E_NULL: return "TRN_E_NULL";
        case TRN_E_SHAPE: return "TRN_E_SHAPE";
        case TRN_E_STRIDE: return "TRN_E_STRIDE";
        case TRN_E_ALIGN: return "TRN_E_ALIGN";
        case TRN_E_UNSUPPORTED: return "TRN_E_UNSUPPORTED";
        case TRN_E_LAUNCH: return "TRN_E_LAUNCH";
        case TRN_E_ARCH: return "TRN_E_ARCH";
        default: return "TRN_E_UNKNOWN";
    }
}

extern "C" int trn_check_device(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return TRN_E_ARCH;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return TRN_E_ARCH;
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? TRN_OK : TRN_E_ARCH;
}

// Plain streaming copy, 16 bytes per lane, non-temporal both ways: the yardstick that HBM counters and
// achieved bandwidth of the real kernels are calibrated against.
namespace trn {
__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4_t* __restrict__ src, uint4_t* __restrict__ dst,
                                                               int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}
}  // namespace trn

extern "C" int trn_calibration_copy(const void* src, void* dst, int64_t bytes, void* stream) {
    using namespace trn;
    if (bytes < 0 || bytes % 16) return TRN_E_SHAPE;
    if (bytes == 0) return TRN_OK;
    if (!src || !dst) return TRN_E_NULL;
    if (!aligned16(src) || !aligned16(dst)) return TRN_E_ALIGN;
    const int64_t n16 = bytes / 16, grid = (n16 + 255) / 256;
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    hipLaunchKernelGGL(calibration_copy_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                       (const uint4_t*)src, (uint4_t*)dst, n16);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
