// Shared device helpers for the gfx950 kernels: vector types, MFMA wrappers, wave utilities.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/trinity_hip.h"

namespace trn {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// D(32x32) += A(32x16) * B(16x32), fp16 in, fp32 out.  Lane l supplies A[l%32][8*(l/32)..+7]
// and B[8*(l/32)..+7][l%32]; it receives D[8*(r/4) + 4*(l/32) + r%4][l%32] in element r.
__device__ __forceinline__ float16_t mfma32(half8_t a, half8_t b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// Combine a value with the one held by the lane 32 away (the other half of a 32x32 accumulator
// column).  v_permlane32_swap exchanges the upper half of one register with the lower half of another:
// starting from two copies of x it leaves {own, other} in the pair (order depends on the lane half), and
// max / + are commutative.  One VALU op, no LDS traffic -- it must not queue behind the LDS operand
// prefetches.  Issued as inline asm: the compiler's builtin for this instruction mis-folds its second
// result when both results feed one operation.  The s_nop covers the VALU-write -> permlane-read hazard.
__device__ __forceinline__ void swap_halves(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float half_max(float x) { float a = x, b = x; swap_halves(a, b); return fmaxf(a, b); }
__device__ __forceinline__ float half_sum(float x) { float a = x, b = x; swap_halves(a, b); return a + b; }

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane a points at 4 fp16
// (8 bytes); lanes 4r..4r+3 together supply "row" r = 16 consecutive elements (their addresses need
// not be adjacent in memory, only their order matters).  Lane i of the group receives element i of
// rows 0..3.  With a row-major [k][n] tile in LDS this hands every lane 4 consecutive k for one n,
// i.e. an MFMA operand whose contraction index runs down the tile's rows.
typedef __fp16 fp16x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4_t lds_read_tr16(const half_t* p) {
    fp16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
        (fp16x4_t __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(half4_t, r);
}

// max of 16 values in 8 three-input maxima (v_max3_f32) instead of a chain of 15 two-input ones
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
__device__ __forceinline__ float max16(const float16_t& s) {
    const float a = max3(s[0], s[1], s[2]), b = max3(s[3], s[4], s[5]), c = max3(s[6], s[7], s[8]);
    const float d = max3(s[9], s[10], s[11]), e = max3(s[12], s[13], s[14]);
    return fmaxf(max3(a, b, s[15]), max3(c, d, e));
}

// The same maximum issued as the bare instructions.  fmaxf on a value the compiler cannot prove to be no signalling
// NaN (an MFMA result, a value that passed a select) is preceded by a canonicalising v_max_f32 x, x, x: 15 extra
// instructions per 16 values.  The hardware maximum quiets NaNs by itself.  Only for values that were produced at least
// one MFMA earlier: the compiler does not see which registers the instruction reads, so it inserts no wait states
// between a matrix instruction and this read of its result.
__device__ __forceinline__ float max3_bare(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max16_bare(const float16_t& s) {
    const float a = max3_bare(s[0], s[1], s[2]), b = max3_bare(s[3], s[4], s[5]), c = max3_bare(s[6], s[7], s[8]);
    const float d = max3_bare(s[9], s[10], s[11]), e = max3_bare(s[12], s[13], s[14]);
    const float x = max3_bare(a, b, s[15]), y = max3_bare(c, d, e);
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    half2_t h = {(half_t)a, (half_t)b};
    return __builtin_bit_cast(uint32_t, h);
}

// XOR swizzle of the 16-byte chunk index within a tile row, as a function of the row.  Tiles are stored
// UNPADDED (direct global->LDS loads write 1 KB contiguous per wave instruction), so bank spreading comes from
// the swizzle: it is a bit permutation of the row's low bits chosen so that (a) 16 consecutive rows read at one
// logical chunk (the K operand: one 16-byte read per lane, lane = row) and (b) 4 consecutive rows read over 4
// consecutive chunks (one phase of the transposing V read) both touch every LDS bank exactly once.
template <int D> __device__ __forceinline__ int swz(int r) {
    if constexpr (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);            // 16 chunks per 256-byte row
    else return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);                        // 8 chunks per 128-byte row
}

// One wave's share of a K or V stage: NI wave-wide 1 KB loads, global -> LDS without passing through
// registers.  Load n covers stage rows n*NW*RPI + wave*RPI + lane/CPR (RPI rows of CPR 16-byte chunks); lane i's
// 16 bytes land at the LDS address of that row group + 16*i.  Which global chunk a lane fetches (vo) decides
// the swizzle; because the row groups of successive loads are a multiple of 16 rows apart the swizzle is the
// same for all of them, so ONE per-lane offset serves every load and the rest is wave-uniform (soffset).
#if defined(__HIP_DEVICE_COMPILE__)
template <int NI, int D, int NW>
__device__ __forceinline__ void fetch_tile(__amdgpu_buffer_rsrc_t rs, half_t* dst_wave, int vo, int soff, int row_step_bytes) {
    constexpr int RPI = 64 / (D / 8);
#pragma unroll
    for (int n = 0; n < NI; ++n)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(dst_wave + n * NW * RPI * D),
                                                 16, vo, soff + n * NW * row_step_bytes, 0, 0);
}
#endif

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool pitch16(int64_t elems, int elem_bytes) { return ((elems * elem_bytes) & 15) == 0; }

}  // namespace trn
