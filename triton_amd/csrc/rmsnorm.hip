// RMSNorm over rows of fp16 data: one pass, the row held in registers between the mean-square
// reduction and the scale.  HBM-bound: 16-byte loads, LPR lanes cooperate on one row and reduce
// with cross-lane shuffles; rows*cols*2 bytes read, the same written.
#include "common.h"

namespace trn {

// LPR lanes per row (power of two <= 64), NV 16-byte vectors per lane.
template <int LPR, int NV>
__global__ __launch_bounds__(256) void rmsnorm_kernel(
    const half_t* x, const half_t* __restrict__ gamma, half_t* y,     // y may be x (in place): a row is read whole
                                                                     // into registers before any of it is written
    int64_t n_rows, int64_t inner_rows, int cols,
    int64_t x_outer, int64_t ldx, int64_t y_outer, int64_t ldy, int64_t row_start, float eps) {
    constexpr int ROWS_PER_BLOCK = 256 / LPR;
    const int sub = threadIdx.x % LPR;
    const uint32_t row = blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / LPR;
    if (row >= (uint32_t)n_rows) return;             // whole LPR-lane groups leave together
    // 32-bit row arithmetic: the address must be ready before the first load can issue, and a 64-bit
    // division on that path costs more than the whole streaming loop of a short row
    uint32_t outer = 0, inner = row;
    if (inner_rows != n_rows) { outer = row / (uint32_t)inner_rows; inner = row - outer * (uint32_t)inner_rows; }
    const half_t* xr = x + (int64_t)outer * x_outer + ((int64_t)inner + row_start) * ldx;
    half_t* yr = y + (int64_t)outer * y_outer + ((int64_t)inner + row_start) * ldy;

    half8_t v[NV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (i * LPR + sub) * 8;
        if (c < cols) {
            v[i] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(xr + c));   // streamed once: keep it out of the caches' way
#pragma unroll
            for (int e = 0; e < 8; ++e) { float f = (float)v[i][e]; ss += f * f; }
        }
    }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    const float rstd = 1.0f / __builtin_sqrtf(ss / (float)cols + eps);

#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (i * LPR + sub) * 8;
        if (c < cols) {
            half8_t o;
            if (gamma) {
                half8_t g = *reinterpret_cast<const half8_t*>(gamma + c);
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)g[e] * ((float)v[i][e] * rstd));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)v[i][e] * rstd);
            }
            __builtin_nontemporal_store(o, reinterpret_cast<half8_t*>(yr + c));
        }
    }
}

template <int LPR, int NV>
static hipError_t launch(const void* x, const void* gamma, void* y, int64_t n_rows, int64_t inner_rows,
                         int cols, int64_t xo, int64_t ldx, int64_t yo, int64_t ldy, int64_t row_start,
                         float eps, hipStream_t s) {
    constexpr int RPB = 256 / LPR;
    dim3 grid((unsigned)((n_rows + RPB - 1) / RPB));
    hipLaunchKernelGGL((rmsnorm_kernel<LPR, NV>), grid, dim3(256), 0, s, (const half_t*)x,
                       (const half_t*)gamma, (half_t*)y, n_rows, inner_rows, cols, xo, ldx, yo, ldy,
                       row_start, eps);
    return hipGetLastError();
}

}  // namespace trn

extern "C" int trn_rmsnorm_f16(const void* x, const void* gamma, void* y, int64_t outer_rows,
                               int64_t inner_rows, int64_t cols, int64_t x_outer_stride, int64_t ldx,
                               int64_t y_outer_stride, int64_t ldy, int64_t row_start, float eps,
                               void* stream) {
    using namespace trn;
    if (outer_rows < 0 || inner_rows < 0 || cols <= 0 || row_start < 0) return TRN_E_SHAPE;
    if (outer_rows * inner_rows == 0) return TRN_OK;      // nothing to do; empty tensors have no storage
    if (!x || !y) return TRN_E_NULL;
    if (cols % 8 != 0 || cols > 16384) return TRN_E_SHAPE;
    if (ldx < cols || ldy < cols) return TRN_E_STRIDE;
    if (!aligned16(x) || !aligned16(y) || (gamma && !aligned16(gamma))) return TRN_E_ALIGN;
    if (!pitch16(ldx, 2) || !pitch16(ldy, 2) || !pitch16(x_outer_stride, 2) || !pitch16(y_outer_stride, 2))
        return TRN_E_ALIGN;
    const int64_t n_rows = outer_rows * inner_rows;
    if (n_rows == 0) return TRN_OK;
    if (n_rows > (int64_t)0x7fffffff) return TRN_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const int vecs = (int)(cols / 8);
    hipError_t e;
#define TRN_RMS(LPR, NV) e = launch<LPR, NV>(x, gamma, y, n_rows, inner_rows, (int)cols, x_outer_stride, ldx, y_outer_stride, ldy, row_start, eps, s)
    if (vecs <= 8) TRN_RMS(8, 1);
    else if (vecs <= 16) TRN_RMS(16, 1);
    else if (vecs <= 32) TRN_RMS(32, 1);
    else if (vecs <= 64) TRN_RMS(64, 1);
    else if (vecs <= 128) TRN_RMS(64, 2);
    else if (vecs <= 256) TRN_RMS(64, 4);
    else if (vecs <= 512) TRN_RMS(64, 8);
    else if (vecs <= 1024) TRN_RMS(64, 16);
    else TRN_RMS(64, 32);
#undef TRN_RMS
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
