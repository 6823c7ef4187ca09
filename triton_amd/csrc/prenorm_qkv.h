// Argument block shared by the two tile shapes of the fused RMSNorm + Q/K/V projection GEMM.
#pragma once
#include "common.h"

namespace trn {

// One projection: weight [hidden][n] with row pitch ldw, head-split output, and the index of its first
// column panel in the concatenated [Q | K | V] panel list.
struct ProjOut { const half_t* w; half_t* out; int64_t ldw, stride_h, stride_s; int n; int tile0; };

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
int launch_prenorm_qkv_wide(GemmArgs a, int64_t n_q, int64_t n_kv, hipStream_t stream);
int64_t prenorm_qkv_wide_tiles(int64_t tokens, int64_t n_q, int64_t n_kv);

// At most 32 tokens: 64-column panels streamed by four waves that split the contraction (prenorm_qkv_skinny.hip).
int launch_prenorm_qkv_skinny(GemmArgs a, int64_t n_q, int64_t n_kv, hipStream_t stream);

}  // namespace trn
