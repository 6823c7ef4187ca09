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
// lane ends up with 4 consecutive output columns of ONE token (one rstd per lane).  W is [hidden][n] row-major
// with the contraction index running down its rows: its tiles go straight from global memory into LDS
// (buffer_load ... lds), row-major with an XOR chunk swizzle, and the W^T A-operand is fetched with the
// transposing LDS read ds_read_b64_tr_b16.  X^T is the B operand (16-byte reads of a padded tile that was
// written from registers).  256 threads = 4 waves in a 2x2 arrangement, each wave a 64x64 sub-tile.  Both
// tiles are double-buffered: the W fetch and the X global loads of k-tile j+1 are issued before the MFMAs of
// k-tile j, one barrier per k-tile.  The epilogue transposes each wave's tile through LDS so that the stores
// are whole 16-byte-per-lane row segments.
#include "prenorm_qkv.h"

namespace trn {

[[maybe_unused]] constexpr int GBM = 128, GBN = 128, GBK = 64;

__global__ __launch_bounds__(256, 2) void prenorm_qkv_kernel(const GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    constexpr int XP = GBK + 8;    // X tile pitch (halfs): rows 36 banks apart -> conflict-free 16-byte row reads
    // separate arrays per stage: the compiler orders LDS reads after outstanding global->LDS loads that may
    // alias them, and only distinct variables are provably disjoint
    __shared__ __attribute__((aligned(1024))) half_t Ws0[GBK * GBN];
    __shared__ __attribute__((aligned(1024))) half_t Ws1[GBK * GBN];
    __shared__ __attribute__((aligned(16))) half_t Xs0[GBM * XP];
    __shared__ __attribute__((aligned(16))) half_t Xs1[GBM * XP];
    __shared__ float rstd_s[GBM];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;

    // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  XCD x owns a contiguous run of
    // 128-column panels of W and walks the token tiles fastest, so the workgroups resident on it together
    // share a few W panels and each X slab between them instead of every XCD streaming all of W and X.
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int mt = local % a.n_mtiles, nt_all = xcd * a.panels_per_xcd + local / a.n_mtiles;
    if (nt_all >= a.n_panels) return;
    const int pi = nt_all >= a.p[2].tile0 ? 2 : (nt_all >= a.p[1].tile0 ? 1 : 0);
    const ProjOut P = a.p[pi];
    const int n0 = (nt_all - P.tile0) * GBN, m0 = mt * GBM;

    // ---- W: direct global -> LDS.  One wave-wide load covers 4 rows of 256 bytes; load i of this wave covers
    // stage rows 16*i + 4*wave + lane/16, so the swizzle (a function of row % 16) is the same for all four
    // and one per-lane offset serves them.
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)P.w, 0, (int)(((int64_t)(a.K - 1) * P.ldw + P.n) * 2), 0x00020000);
    const int w_row = 4 * wave + lane / 16;
    const int w_vo = (int)(w_row * P.ldw * 2) + (n0 + (((lane & 15) ^ wswz(w_row)) << 3)) * 2;
    const int w_row16 = (int)(16 * P.ldw * 2), w_tile = (int)(GBK * P.ldw * 2);
#define TRN_FETCH_W(kt_, dst_)                                                                                   \
    _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) __builtin_amdgcn_raw_ptr_buffer_load_lds(                  \
        wrs, (__attribute__((address_space(3))) void*)(&dst_[(16 * i_ + 4 * wave) * GBN]), 16, w_vo,             \
        (kt_) * w_tile + i_ * w_row16, 0, 0)

    // ---- X: global -> registers (gamma, sum of squares) -> LDS.  Thread covers rows xr + 32*i, 8 halfs at xc.
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)a.x, 0, (int)(((int64_t)(a.T - 1) * a.ldx + a.K) * 2), 0x00020000);
    const int xr = tid >> 3, xc = (tid & 7) * 8;
    int x_vo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = m0 + xr + 32 * i;
        x_vo[i] = t < a.T ? (int)(t * a.ldx * 2) + xc * 2 : 0x7ffffff0;     // rows past the end: out of range -> zeros
    }
    uint4_t xreg[4];
    half8_t greg = {0, 0, 0, 0, 0, 0, 0, 0};
    float ss[4] = {0.f, 0.f, 0.f, 0.f};
    const bool use_g = a.gamma != nullptr && a.norm;
    const bool ragged_k = (a.K % GBK) != 0;
    auto fetch_x = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) xreg[i] = __builtin_amdgcn_raw_buffer_load_b128(xrs, x_vo[i], kt * GBK * 2, 0);
        if (use_g) greg = kt * GBK + xc < a.K ? *reinterpret_cast<const half8_t*>(a.gamma + kt * GBK + xc) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    };
    // Packed fp16 arithmetic keeps this off the critical path (the MFMAs of a k-tile take 512 cycles per wave):
    // x*gamma as one fp16 multiply per pair is the correctly rounded product, i.e. what an fp32 multiply rounded
    // to fp16 gives, and the squares are summed two at a time into fp32 by the dot-product instruction.
    auto stash_x = [&](int kt, half_t* Xd) __attribute__((always_inline)) {
        // columns past hidden hold the next row's data: ignore them (only the last k-tile can have any)
        const bool drop = ragged_k && kt * GBK + xc >= a.K;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            half8_t xv = __builtin_bit_cast(half8_t, xreg[i]);
            if (ragged_k) { if (drop) xv = half8_t{0, 0, 0, 0, 0, 0, 0, 0}; }
            if (a.norm) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const half2_t p = {xv[2 * e], xv[2 * e + 1]};
                    ss[i] = __builtin_amdgcn_fdot2(p, p, ss[i], false);
                }
                if (use_g) xv = xv * greg;
            }
            *reinterpret_cast<half8_t*>(&Xd[(xr + 32 * i) * XP + xc]) = xv;
        }
    };

    // ---- LDS read offsets (halfs).  X^T B-operand: row wm*64 + mb*32 + c, columns ks*16 + 8h.
    const int xoff = (wm * 64 + c) * XP + 8 * h;
    // W^T A-operand via the transposing read: lane's piece is stage row ks*16 + 8h + (lane%16)/4 [+4], columns
    // wn*64 + nb*32 + 16*((lane/16)%2) + 4*(lane%4)
    int woff_lo[2], woff_hi[2];
    {
        const int rl = 8 * h + ((lane & 15) >> 2), rh = rl + 4;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int chunk = wn * 8 + nb * 4 + lc;
            woff_lo[nb] = rl * GBN + ((chunk ^ wswz(rl)) << 3) + sub;
            woff_hi[nb] = rh * GBN + ((chunk ^ wswz(rh)) << 3) + sub;
        }
    }

    float16_t acc[2][2];   // [n block][m block]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jn = 0; jn < 2; ++jn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

    const int nk = (a.K + GBK - 1) / GBK;
    TRN_FETCH_W(0, Ws0);
    fetch_x(0);
    stash_x(0, Xs0);
    __builtin_amdgcn_s_waitcnt(0x0f70);     // vmcnt(0)
    __syncthreads();

    auto ktile = [&](int kt, const half_t* Wc, const half_t* Xc, half_t* Wn, half_t* Xn) __attribute__((always_inline)) {
        const bool more = kt + 1 < nk;
        if (more) { TRN_FETCH_W(kt + 1, Wn); fetch_x(kt + 1); }      // land during the MFMAs below
#pragma unroll
        for (int ks = 0; ks < GBK / 16; ++ks) {
            half8_t xb[2], wa[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
                xb[mb] = *reinterpret_cast<const half8_t*>(&Xc[xoff + mb * 32 * XP + ks * 16]);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                half4_t lo = lds_read_tr16(&Wc[ks * 16 * GBN + woff_lo[nb]]);
                half4_t hi = lds_read_tr16(&Wc[ks * 16 * GBN + woff_hi[nb]]);
                wa[nb] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) acc[nb][mb] = mfma32(wa[nb], xb[mb], acc[nb][mb]);
        }
        if (more) stash_x(kt + 1, Xn);            // nobody reads Xn: its last readers passed the previous barrier
        __builtin_amdgcn_s_waitcnt(0x0f70);       // vmcnt(0): this wave's share of the next W stage is in LDS
        __syncthreads();
    };
    for (int kt = 0; kt < nk; kt += 2) {
        ktile(kt, Ws0, Xs0, Ws1, Xs1);
        if (kt + 1 < nk) ktile(kt + 1, Ws1, Xs1, Ws0, Xs0);
    }
#undef TRN_FETCH_W

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

    // ---- epilogue: scale, transpose this wave's 64 x 64 tile through LDS (stage memory is free now), store
    // 16 bytes per lane: 8 lanes cover the 64 columns of a token, 8 tokens per store instruction
    {
        constexpr int OP = 64 + 4;                          // pitch in halfs
        half_t* ot = (wave == 0 ? Ws0 : wave == 1 ? Ws1 : wave == 2 ? Xs0 : Xs1);   // 64*68*2 = 8704 bytes <= a stage
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            const float r = a.norm ? rstd_s[wm * 64 + mb * 32 + c] : 1.0f;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    half4_t ov;
#pragma unroll
                    for (int e = 0; e < 4; ++e) ov[e] = (half_t)(acc[nb][mb][r4 * 4 + e] * r);
                    *reinterpret_cast<half4_t*>(&ot[(mb * 32 + c) * OP + nb * 32 + 8 * r4 + 4 * h]) = ov;
                }
        }
        // (LDS operations of one wave execute in order: its reads below see its writes above)
        const int orow = lane >> 3, ocol = (lane & 7) * 8;
        const int n = n0 + wn * 64 + ocol;
        const int64_t o_off = (int64_t)(n / a.head_dim) * P.stride_h + (n % a.head_dim);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int tl = j * 8 + orow, t = m0 + wm * 64 + tl;
            const half4_t lo = *reinterpret_cast<const half4_t*>(&ot[tl * OP + ocol]);
            const half4_t hi = *reinterpret_cast<const half4_t*>(&ot[tl * OP + ocol + 4]);
            half8_t ov = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            if (t < a.T && n < P.n) {
                if (P.addend) {
                    const half8_t ad = *reinterpret_cast<const half8_t*>(P.addend + o_off + (int64_t)t * P.stride_s);
#pragma unroll
                    for (int e = 0; e < 8; ++e) ov[e] = (half_t)((float)ov[e] + (float)ad[e]);
                }
                *reinterpret_cast<half8_t*>(P.out + o_off + (int64_t)t * P.stride_s) = ov;
            }
        }
    }
#endif
}

// The tiling is chosen by problem size.
int launch_projections(GemmArgs a, hipStream_t stream) {
    // a handful of tokens (decode): the weight stream is everything
    if (a.T <= 32) return launch_prenorm_qkv_skinny(a, stream);
    // 256-token tiles once they alone occupy at least half of the 256 CUs; 128 x 128 tiles below that (short
    // prefills, where the number of workgroups matters more than the work per staged byte)
    if (prenorm_qkv_wide_tiles(a) >= 128) return launch_prenorm_qkv_wide(a, stream);
    a.n_mtiles = (a.T + GBM - 1) / GBM;
    int t0 = 0;
    for (int i = 0; i < 3; ++i) { a.p[i].tile0 = t0; t0 += (a.p[i].n + GBN - 1) / GBN; }
    a.n_panels = t0;
    a.panels_per_xcd = (a.n_panels + 7) / 8;
    const int64_t grid = (int64_t)8 * a.panels_per_xcd * a.n_mtiles;
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    hipLaunchKernelGGL(prenorm_qkv_kernel, dim3((unsigned)grid), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}

// out = act(c1) * c2, elementwise over [rows, cols] fp16 (the gate of a gated MLP); 8 columns per lane
__global__ __launch_bounds__(256) void gate_kernel(const half_t* c1, const half_t* c2, half_t* out, int64_t rows, int cols,
                                                   int64_t ld1, int64_t ld2, int64_t ldo, int silu) {
    const int chunks = cols / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * chunks) return;
    const int64_t r = i / chunks; const int cc = (int)(i % chunks) * 8;
    const half8_t u = *reinterpret_cast<const half8_t*>(c1 + r * ld1 + cc), v = *reinterpret_cast<const half8_t*>(c2 + r * ld2 + cc);
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float x = (float)u[e], sg = 1.0f / (1.0f + fast_exp2(-x * kLog2e));
        o[e] = (half_t)((silu ? x * sg : sg) * (float)v[e]);
    }
    *reinterpret_cast<half8_t*>(out + r * ldo + cc) = o;
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
    const int64_t pitches[] = {ldx, ldwq, ldwk, ldwv, q_stride_h, q_stride_s, k_stride_h, k_stride_s, v_stride_h, v_stride_s};
    for (int64_t p : pitches) if (!pitch16(p, 2)) return TRN_E_ALIGN;     // 16-byte loads and stores
    // X and W tiles are fetched with 32-bit buffer offsets
    // (with room for the tiles the pipelines request past the end, which must stay representable to read as zeros)
    const int64_t spans[] = {(tokens + 256) * ldx * 2, (hidden + 512) * ldwq * 2, (hidden + 512) * ldwk * 2, (hidden + 512) * ldwv * 2};
    for (int64_t sp : spans) if (sp > 0x7fffffffLL) return TRN_E_UNSUPPORTED;

    GemmArgs a;
    a.x = (const half_t*)x; a.gamma = (const half_t*)gamma;
    a.T = (int)tokens; a.K = (int)hidden; a.head_dim = (int)head_dim; a.ldx = ldx; a.eps = eps; a.norm = norm ? 1 : 0;
    a.p[0] = ProjOut{(const half_t*)wq, (half_t*)q, ldwq, q_stride_h, q_stride_s, (int)n_q, 0, nullptr};
    a.p[1] = ProjOut{(const half_t*)wk, (half_t*)k, ldwk, k_stride_h, k_stride_s, (int)n_kv, 0, nullptr};
    a.p[2] = ProjOut{(const half_t*)wv, (half_t*)v, ldwv, v_stride_h, v_stride_s, (int)n_kv, 0, nullptr};
    return launch_projections(a, (hipStream_t)stream);
}

extern "C" int trn_linear_f16(const void* x, int64_t tokens, int64_t hidden, int64_t ldx, int32_t n_mats,
                              const void* const* w, const int64_t* n, const int64_t* ldw, void* const* out,
                              const int64_t* ldo, const void* const* addend, void* stream) {
    using namespace trn;
    if (tokens < 0 || hidden <= 0 || n_mats < 1 || n_mats > 3) return TRN_E_SHAPE;
    if (!x || !w || !n || !ldw || !out || !ldo) return TRN_E_NULL;
    if (tokens == 0) return TRN_OK;
    if (hidden % 8 || tokens > 0x7fffffff || hidden > 0x7fffffff) return TRN_E_SHAPE;
    if (ldx < hidden) return TRN_E_STRIDE;
    if (!aligned16(x) || !pitch16(ldx, 2)) return TRN_E_ALIGN;
    if ((tokens + 256) * ldx * 2 > 0x7fffffffLL) return TRN_E_UNSUPPORTED;
    GemmArgs a;
    a.x = (const half_t*)x; a.gamma = nullptr;
    a.T = (int)tokens; a.K = (int)hidden; a.ldx = ldx; a.eps = 0.f; a.norm = 0;
    // plain row-major outputs [tokens, n_i]: "heads" of 8 columns at a pitch of 8 put column n at offset n
    a.head_dim = 8;
    for (int i = 0; i < 3; ++i) a.p[i] = ProjOut{nullptr, nullptr, 0, 0, 0, 0, 0, nullptr};
    for (int i = 0; i < n_mats; ++i) {
        if (!w[i] || !out[i]) return TRN_E_NULL;
        if (n[i] <= 0 || n[i] % 8 || n[i] > 0x7fffffff) return TRN_E_SHAPE;
        if (ldw[i] < n[i] || ldo[i] < n[i]) return TRN_E_STRIDE;
        const void* ad = addend ? addend[i] : nullptr;
        if (!aligned16(w[i]) || !aligned16(out[i]) || (ad && !aligned16(ad)) || !pitch16(ldw[i], 2) || !pitch16(ldo[i], 2)) return TRN_E_ALIGN;
        if ((hidden + 512) * ldw[i] * 2 > 0x7fffffffLL) return TRN_E_UNSUPPORTED;
        a.p[i] = ProjOut{(const half_t*)w[i], (half_t*)out[i], ldw[i], 8, ldo[i], (int)n[i], 0, (const half_t*)ad};
    }
    return launch_projections(a, (hipStream_t)stream);
}

extern "C" int trn_gate_f16(const void* c1, const void* c2, void* out, int64_t rows, int64_t cols, int64_t ld1,
                            int64_t ld2, int64_t ldo, int32_t kind, void* stream) {
    using namespace trn;
    if (rows < 0 || cols <= 0 || cols % 8 || cols > 0x7fffffff || (kind != 0 && kind != 1)) return TRN_E_SHAPE;
    if (rows == 0) return TRN_OK;
    if (!c1 || !c2 || !out) return TRN_E_NULL;
    if (ld1 < cols || ld2 < cols || ldo < cols) return TRN_E_STRIDE;
    if (!aligned16(c1) || !aligned16(c2) || !aligned16(out) || !pitch16(ld1, 2) || !pitch16(ld2, 2) || !pitch16(ldo, 2)) return TRN_E_ALIGN;
    const int64_t work = rows * (cols / 8), grid = (work + 255) / 256;
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    hipLaunchKernelGGL(gate_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (const half_t*)c1, (const half_t*)c2,
                       (half_t*)out, rows, (int)cols, ld1, ld2, ldo, kind);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
