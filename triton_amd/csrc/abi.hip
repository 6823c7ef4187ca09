// Library-level entry points: version, status names, device check.
#include "attn.h"
#include <string.h>

extern "C" int trn_version(void) { return 300; }  // 0.3.0: minor number = count of ABI revisions (entry points added)

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
        case TRN_E_SCRATCH: return "TRN_E_SCRATCH";
        default: return "TRN_E_UNKNOWN";
    }
}

extern "C" int trn_check_device(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return TRN_E_ARCH;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return TRN_E_ARCH;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return TRN_E_ARCH;
    // set-up that must not happen under graph capture: the address of the static scratch array on this device
    return trn::attn_static_scratch() ? TRN_OK : TRN_E_LAUNCH;
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

// Nothing but back-to-back v_mfma_f32_32x32x16_f16 from registers (8 operand pairs per lane taken from
// `operands`, 4 accumulators): what the matrix pipes sustain on this board for a given operand data pattern.
// With all-zero operands it runs at the nominal rate; with random operands the board's power limit pulls the
// clock down -- the ceiling any MFMA-bound kernel on real data is measured against.
namespace trn {
__global__ __launch_bounds__(256) void calibration_mfma_kernel(const half8_t* __restrict__ operands, float* __restrict__ sink,
                                                               int iters) {
    half8_t a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = operands[threadIdx.x + 256 * i]; b[i] = operands[threadIdx.x + 256 * (8 + i)]; }
    float16_t c0, c1, c2, c3;
#pragma unroll
    for (int e = 0; e < 16; ++e) { c0[e] = 0.f; c1[e] = 0.f; c2[e] = 0.f; c3[e] = 0.f; }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; j += 4) {
            c0 = mfma32(a[j], b[j], c0); c1 = mfma32(a[j + 1], b[j + 1], c1);
            c2 = mfma32(a[j + 2], b[j + 2], c2); c3 = mfma32(a[j + 3], b[j + 3], c3);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) s += c0[e] + c1[e] + c2[e] + c3[e];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}
}  // namespace trn

extern "C" int trn_calibration_mfma(const void* operands, float* sink, int32_t iters, int32_t n_workgroups, void* stream) {
    using namespace trn;
    if (iters <= 0 || n_workgroups <= 0) return TRN_E_SHAPE;
    if (!operands || !sink) return TRN_E_NULL;
    if (!aligned16(operands)) return TRN_E_ALIGN;
    hipLaunchKernelGGL(calibration_mfma_kernel, dim3((unsigned)n_workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const half8_t*)operands, sink, iters);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
