// Argument block shared by the two tile shapes of the fused RMSNorm + Q/K/V projection GEMM.
#pragma once
#include "common.h"

namespace trn {

// One projection: weight [hidden][n] with row pitch ldw, head-split output, the index of its first column panel in
// the concatenated [Q | K | V] panel list, and an optional addend laid out like the output (out = x w + addend; it
// may be the output itself).  n = 0: no such projection.
struct ProjOut { const half_t* w; half_t* out; int64_t ldw, stride_h, stride_s; int n; int tile0; const half_t* addend; };

// Panels are GBN (128) or WN (256) columns wide depending on the kernel; n_mtiles counts token tiles likewise.
struct GemmArgs {
    const half_t* x; const half_t* gamma;
    ProjOut p[3];
    int T, K, head_dim, n_mtiles, n_panels, panels_per_xcd;
    int64_t ldx;
    float eps;
    int norm;
};

// Chunk swizzle of a W stage row (16-byte chunks) as a function of the row: a bit permutation of the row's low
// 4 bits, XORed into the low 4 bits of the chunk index, under which 4 consecutive rows read over 4 consecutive
// chunks (one phase of the transposing read) touch every bank once.
__device__ __forceinline__ int wswz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

// 256 x 256 workgroup tiles, for problems large enough to fill the chip with them (prenorm_qkv_wide.hip).
int launch_prenorm_qkv_wide(GemmArgs a, hipStream_t stream);
int64_t prenorm_qkv_wide_tiles(const GemmArgs& a);

// At most 32 tokens: 64-column panels streamed by four waves that split the contraction (prenorm_qkv_skinny.hip).
int launch_prenorm_qkv_skinny(GemmArgs a, hipStream_t stream);

// The 128 x 128 tiling and the choice between the three (prenorm_qkv.hip).
int launch_projections(GemmArgs a, hipStream_t stream);

}  // namespace trn
