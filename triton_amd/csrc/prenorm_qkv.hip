// Fused RMSNorm + Q/K/V projection GEMM for gfx950.
//
//     Q|K|V[t][n] = rstd[t] * sum_k (x[t][k] * gamma[k]) * W[k][n],   rstd[t] = rsqrt(mean_k x[t][k]^2 + eps)
//
// The normalisation never makes its own pass over X: the workgroup that computes a 128-token x 128-column
// output tile streams the whole 128 x hidden slab of X through its registers on the way to LDS anyway, so it
// accumulates the row sums of squares there, multiplies by gamma at the same point, and applies rstd as a
// row scale to the fp32 accumulator at the end ((x*r)@W == r*(x@W)).
//
// MFMA mapping (32x32x16 fp16): the product is formed transposed, C^T[n][t] = W^T[n][k] X^T[k][t], so that a
// lane ends up with 4 consecutive output columns of ONE token (8-byte stores, one rstd per lane).  W is
// [hidden][n] row-major with the contraction index running down its rows; the W^T A-operand is fetched from
// the row-major LDS tile with the transposing read ds_read_b64_tr_b16.  X^T is the B operand (16-byte reads).
// 256 threads = 4 waves in a 2x2 arrangement, each wave a 64x64 sub-tile; global loads for the next k-tile
// are issued into registers before the MFMAs of the current one.
#include "common.h"

namespace trn {

struct ProjOut { const half_t* w; half_t* out; int64_t ldw, stride_h, stride_s; int n; int tile0; };

struct GemmArgs {
    const half_t* x; const half_t* gamma;
    ProjOut p[3];
    int T, K, head_dim, n_mtiles;
    int64_t ldx;
    float eps;
    int norm;
};

constexpr int GBM = 128, GBN = 128, GBK = 64;

__global__ __launch_bounds__(256, 2) void prenorm_qkv_kernel(const GemmArgs a) {
    constexpr int XP = GBK + 8;    // X tile pitch (halfs)
    constexpr int WP = GBN + 8;    // W tile pitch (halfs)
    __shared__ __attribute__((aligned(16))) half_t Xs[GBM * XP];
    __shared__ __attribute__((aligned(16))) half_t Ws[GBK * WP];
    __shared__ float rstd_s[GBM];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wm = wave & 1, wn = wave >> 1;
    const int tr_row = (lane & 15) >> 2, tr_col = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;

    const int mt = blockIdx.x % a.n_mtiles, nt_all = blockIdx.x / a.n_mtiles;
    const int pi = nt_all >= a.p[2].tile0 ? 2 : (nt_all >= a.p[1].tile0 ? 1 : 0);
    const ProjOut P = a.p[pi];
    const int n0 = (nt_all - P.tile0) * GBN, m0 = mt * GBM;

    // fixed per-thread staging coordinates
    const int xr = tid >> 3, xc = (tid & 7) * 8;       // X: rows xr + 32*i, 8 halfs at column xc
    const int wr = tid >> 4, wc = (tid & 15) * 8;      // W: rows wr + 16*i, 8 halfs at column wc
    uint4_t xreg[4], wreg[4];
    float ss[4] = {0.f, 0.f, 0.f, 0.f};

    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = m0 + xr + 32 * i, k = k0 + xc;
            xreg[i] = uint4_t{0u, 0u, 0u, 0u};
            if (t < a.T && k < a.K) xreg[i] = *reinterpret_cast<const uint4_t*>(a.x + (int64_t)t * a.ldx + k);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + wr + 16 * i, n = n0 + wc;
            wreg[i] = uint4_t{0u, 0u, 0u, 0u};
            if (k < a.K && n < P.n) wreg[i] = *reinterpret_cast<const uint4_t*>(P.w + (int64_t)k * P.ldw + n);
        }
    };
    auto stash = [&](int k0) {
        half8_t gv;
        const bool use_g = a.gamma != nullptr && a.norm;
        if (use_g) {
            gv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            if (k0 + xc < a.K) gv = *reinterpret_cast<const half8_t*>(a.gamma + k0 + xc);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            half8_t xv = __builtin_bit_cast(half8_t, xreg[i]);
            if (a.norm) {
#pragma unroll
                for (int e = 0; e < 8; ++e) { const float f = (float)xv[e]; ss[i] += f * f; }
                if (use_g) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) xv[e] = (half_t)((float)xv[e] * (float)gv[e]);
                }
            }
            *reinterpret_cast<half8_t*>(&Xs[(xr + 32 * i) * XP + xc]) = xv;
            *reinterpret_cast<uint4_t*>(&Ws[(wr + 16 * i) * WP + wc]) = wreg[i];
        }
    };

    float16_t acc[2][2];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jn = 0; jn < 2; ++jn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

    const int nk = (a.K + GBK - 1) / GBK;
    fetch(0);
    for (int kt = 0; kt < nk; ++kt) {
        __syncthreads();               // previous tile's MFMAs have read LDS
        stash(kt * GBK);
        __syncthreads();
        if (kt + 1 < nk) fetch((kt + 1) * GBK);   // in flight during the MFMAs below
#pragma unroll
        for (int ks = 0; ks < GBK / 16; ++ks) {
            half8_t xb[2], wa[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
                xb[mb] = *reinterpret_cast<const half8_t*>(&Xs[(wm * 64 + mb * 32 + c) * XP + ks * 16 + 8 * h]);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const half_t* wp = &Ws[(ks * 16 + 8 * h + tr_row) * WP + wn * 64 + nb * 32 + tr_col];
                half4_t lo = lds_read_tr16(wp), hi = lds_read_tr16(wp + 4 * WP);
                wa[nb] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) acc[nb][mb] = mfma32(wa[nb], xb[mb], acc[nb][mb]);
        }
    }

    // row rstd: the 8 threads that staged a row's chunks hold its partial sums of squares
    if (a.norm) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s = ss[i];
            s += __shfl_xor(s, 1, 64); s += __shfl_xor(s, 2, 64); s += __shfl_xor(s, 4, 64);
            if ((tid & 7) == 0) rstd_s[xr + 32 * i] = 1.0f / __builtin_sqrtf(s / (float)a.K + a.eps);
        }
    }
    __syncthreads();

#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const int tl = wm * 64 + mb * 32 + c, t = m0 + tl;
        if (t >= a.T) continue;
        const float r = a.norm ? rstd_s[tl] : 1.0f;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int n = n0 + wn * 64 + nb * 32 + 8 * r4 + 4 * h;
                if (n >= P.n) continue;
                half4_t ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) ov[e] = (half_t)(acc[nb][mb][r4 * 4 + e] * r);
                half_t* dst = P.out + (int64_t)(n / a.head_dim) * P.stride_h + (int64_t)t * P.stride_s + (n % a.head_dim);
                *reinterpret_cast<half4_t*>(dst) = ov;
            }
    }
}

}  // namespace trn

extern "C" int trn_prenorm_qkv_f16(const void* x, const void* gamma, const void* wq, const void* wk, const void* wv,
                                   void* q, void* k, void* v, int64_t tokens, int64_t hidden, int64_t n_q,
                                   int64_t n_kv, int64_t head_dim, int64_t ldx, int64_t ldwq, int64_t ldwk,
                                   int64_t ldwv, int64_t q_stride_h, int64_t q_stride_s, int64_t k_stride_h,
                                   int64_t k_stride_s, int64_t v_stride_h, int64_t v_stride_s, float eps,
                                   int32_t norm, void* stream) {
    using namespace trn;
    if (tokens < 0 || hidden <= 0 || n_q <= 0 || n_kv <= 0 || head_dim <= 0) return TRN_E_SHAPE;
    if (tokens == 0) return TRN_OK;
    if (!x || !wq || !wk || !wv || !q || !k || !v) return TRN_E_NULL;
    if (hidden % 8 || n_q % 8 || n_kv % 8 || head_dim % 8 || n_q % head_dim || n_kv % head_dim) return TRN_E_SHAPE;
    if (tokens > 0x7fffffff || hidden > 0x7fffffff || n_q > 0x7fffffff || n_kv > 0x7fffffff) return TRN_E_SHAPE;
    if (ldx < hidden || ldwq < n_q || ldwk < n_kv || ldwv < n_kv) return TRN_E_STRIDE;
    if (q_stride_s < head_dim || k_stride_s < head_dim || v_stride_s < head_dim) return TRN_E_STRIDE;
    const void* ptrs[] = {x, wq, wk, wv, q, k, v};
    for (const void* p : ptrs) if (!aligned16(p)) return TRN_E_ALIGN;
    if (gamma && !aligned16(gamma)) return TRN_E_ALIGN;
    const int64_t pitches[] = {ldx, ldwq, ldwk, ldwv};
    for (int64_t p : pitches) if (!pitch16(p, 2)) return TRN_E_ALIGN;
    const int64_t ostr[] = {q_stride_h, q_stride_s, k_stride_h, k_stride_s, v_stride_h, v_stride_s};
    for (int64_t p : ostr) if ((p * 2) % 8) return TRN_E_ALIGN;     // 8-byte output stores

    GemmArgs a;
    a.x = (const half_t*)x; a.gamma = (const half_t*)gamma;
    a.T = (int)tokens; a.K = (int)hidden; a.head_dim = (int)head_dim; a.ldx = ldx; a.eps = eps; a.norm = norm ? 1 : 0;
    a.n_mtiles = (int)((tokens + GBM - 1) / GBM);
    const int tq = (int)((n_q + GBN - 1) / GBN), tkv = (int)((n_kv + GBN - 1) / GBN);
    a.p[0] = ProjOut{(const half_t*)wq, (half_t*)q, ldwq, q_stride_h, q_stride_s, (int)n_q, 0};
    a.p[1] = ProjOut{(const half_t*)wk, (half_t*)k, ldwk, k_stride_h, k_stride_s, (int)n_kv, tq};
    a.p[2] = ProjOut{(const half_t*)wv, (half_t*)v, ldwv, v_stride_h, v_stride_s, (int)n_kv, tq + tkv};
    const int64_t grid = (int64_t)a.n_mtiles * (tq + 2 * tkv);
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    hipLaunchKernelGGL(prenorm_qkv_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
