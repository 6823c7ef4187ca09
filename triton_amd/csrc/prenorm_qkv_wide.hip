// Fused RMSNorm + Q/K/V projection GEMM, 256-token x 256-column workgroup tiles (large problems).
//
// Same arithmetic and MFMA mapping as the 128 x 128 kernel (C^T = W^T X^T with 32x32x16 fp16 MFMAs, a lane owns
// one token), re-balanced for what limits a large GEMM on this chip:
//   * 4 waves, one per SIMD, each a 128-token x 128-column sub-tile (4 x 4 MFMA blocks, 256 accumulator
//     registers -- the whole AGPR file of a wave that has its SIMD to itself): every 16-byte LDS operand feeds
//     four MFMAs instead of two, so LDS bytes and LDS instructions per MFMA are halved.
//   * Both operands go straight from global memory into LDS (buffer_load ... lds, XOR-swizzled rows); no
//     register staging and no LDS writes from the VALU.  gamma is multiplied into the X operand after it is read
//     back from LDS (one packed fp16 multiply per pair: the correctly rounded product), and the waves of the
//     first column group also sum its squares with the fp32 dot-product instruction for the row rstd.
//   * Four stages of 32 contraction columns: a stage is requested three k-tiles before its first use,
//     which at 256 x 256 flops per staged column covers the L2 / HBM latency.
//   * The one barrier per k-tile sits between the two 16-column halves of the tile's MFMAs, after the second
//     half's operands are already in registers: waves reach it with MFMAs in flight, and the first operands of
//     the next tile are read right behind it, so neither the barrier nor the LDS latency drains the MFMA pipe.
#include "prenorm_qkv.h"

namespace trn {

[[maybe_unused]] constexpr int WM = 256, WN = 256, WK = 32;

__global__ __launch_bounds__(256, 1) void prenorm_qkv_wide_kernel(const GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    // One array per stage and operand: the compiler orders LDS reads after outstanding global->LDS loads that may
    // alias them, and only distinct variables are provably disjoint.
    __shared__ __attribute__((aligned(1024))) half_t Xs0[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs1[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs2[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs3[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Ws0[WK * WN];
    __shared__ __attribute__((aligned(1024))) half_t Ws1[WK * WN];
    __shared__ __attribute__((aligned(1024))) half_t Ws2[WK * WN];
    __shared__ __attribute__((aligned(1024))) half_t Ws3[WK * WN];
    __shared__ float rstd_s[WM];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;          // 2 token halves x 2 column halves

    // Workgroup ids are dealt round-robin to the 8 XCDs; XCD x owns a contiguous run of column panels and walks
    // the token tiles fastest, so its L2 holds a few W panels and each X slab once.
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int mt = local % a.n_mtiles, nt_all = xcd * a.panels_per_xcd + local / a.n_mtiles;
    if (nt_all >= a.n_panels) return;
    const int pi = nt_all >= a.p[2].tile0 ? 2 : (nt_all >= a.p[1].tile0 ? 1 : 0);
    const ProjOut P = a.p[pi];
    const int n0 = (nt_all - P.tile0) * WN, m0 = mt * WM;
    const int nk = (a.K + WK - 1) / WK;
    constexpr int kOut = 0x7ffffff0;                  // a byte offset past every buffer: the load returns zeros

    // ---- W stage: 32 rows x 512 bytes.  A wave-wide load covers 2 rows; load i of this wave covers stage rows
    // 16*(i/2) + 8*(i%2) + 2*wave + lane/32: the swizzle depends on row % 16, so two per-lane offsets serve the four.
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)P.w, 0, (int)(((int64_t)(a.K - 1) * P.ldw + P.n) * 2), 0x00020000);
    int w_vo[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = 8 * i + 2 * wave + (lane >> 5);
        const int chunk = (lane & 16) | ((lane & 15) ^ wswz(r));
        w_vo[i] = (int)(r * P.ldw * 2) + (n0 + 8 * chunk) * 2;
    }
    const int w_row16 = (int)(16 * P.ldw * 2), w_tile = (int)(WK * P.ldw * 2);
    // ---- X stage: 256 rows x 64 bytes, chunk c of row r stored at position c ^ ((r/4) % 4).  A wave-wide load
    // covers 16 rows; load i of this wave covers rows 64*i + 16*wave + lane/4.
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)a.x, 0, (int)(((int64_t)(a.T - 1) * a.ldx + a.K) * 2), 0x00020000);
    const int x_chunk = (lane & 3) ^ ((lane >> 4) & 3);
    int x_vo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = m0 + 64 * i + 16 * wave + (lane >> 2);
        x_vo[i] = t < a.T ? (int)(t * a.ldx * 2) + x_chunk * 16 : kOut;          // rows past the end read as zeros
    }
    // load pair i_ (one X, one W wave-wide load) of stage kt_; columns past hidden hold the next row's data in
    // X: read zeros instead; W rows past hidden are out of range by themselves
#define TRN_FETCH_ONE(kt_, xd_, wd_, i_)                                                                         \
    do {                                                                                                         \
        const bool drop_ = (kt_) * WK + 8 * x_chunk >= a.K;                                                      \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                                \
            xrs, (__attribute__((address_space(3))) void*)(&xd_[(64 * (i_) + 16 * wave) * WK]), 16,              \
            drop_ ? kOut : x_vo[i_], (kt_) * WK * 2, 0, 0);                                                      \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                                \
            wrs, (__attribute__((address_space(3))) void*)(&wd_[(16 * ((i_) >> 1) + 8 * ((i_) & 1) + 2 * wave) * WN]), \
            16, w_vo[(i_) & 1], (kt_) * w_tile + ((i_) >> 1) * w_row16, 0, 0);                                   \
    } while (0)
#define TRN_FETCH(kt_, xd_, wd_) _Pragma("unroll") for (int fi_ = 0; fi_ < 4; ++fi_) TRN_FETCH_ONE(kt_, xd_, wd_, fi_)

    // ---- gamma: the X^T operand of contraction step ks holds columns kt*32 + ks*16 + 8h .. +7 of its token.
    // Without a gamma the multiplier is 1.0, an exact no-op, so that the loop has one form.
    const bool use_g = a.gamma != nullptr && a.norm;
    const bool stats = a.norm && wn == 0;
    const __amdgpu_buffer_rsrc_t grs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(use_g ? a.gamma : a.x), 0, use_g ? a.K * 2 : 0, 0x00020000);
    const half_t one = (half_t)1.0f;
    half8_t g0[2], g1[2], g2[2], g3[2];               // ring over k-tiles, like the stages
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) g0[ks] = g1[ks] = g2[ks] = g3[ks] = half8_t{one, one, one, one, one, one, one, one};
    auto fetch_g = [&](int kt, half8_t (&g)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)       // columns past hidden: zeros (the X operand is zero there as well)
            g[ks] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(grs, (ks * 16 + 8 * h) * 2, kt * WK * 2, 0));
    };

    // ---- LDS read offsets (halfs).  X^T B-operand: row wm*128 + mb*32 + c, chunk 2*ks + h (swizzled).
    int xoff[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) xoff[ks] = (wm * 128 + c) * WK + (((2 * ks + h) ^ ((c >> 2) & 3)) << 3);
    // W^T A-operand via the transposing read: lane's piece is stage row ks*16 + 8h + (lane%16)/4 [+4], columns
    // wn*128 + nb*32 + 16*((lane/16)%2) + 4*(lane%4)
    int woff_lo[4], woff_hi[4];
    {
        const int rl = 8 * h + ((lane & 15) >> 2), rh = rl + 4;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const int chunk = wn * 16 + nb * 4 + lc;
            woff_lo[nb] = rl * WN + ((chunk ^ wswz(rl)) << 3) + sub;
            woff_hi[nb] = rh * WN + ((chunk ^ wswz(rh)) << 3) + sub;
        }
    }
    half8_t xb0[4], xb1[4], wa0[4], wa1[4];           // operands of the two contraction steps of a k-tile
    auto read_x = [&](const half_t* Xc, int ks, int mb) __attribute__((always_inline)) {
        return *reinterpret_cast<const half8_t*>(&Xc[xoff[ks] + mb * 32 * WK]);
    };
    auto read_w = [&](const half_t* Wc, int ks, int nb) __attribute__((always_inline)) {
        const half4_t lo = lds_read_tr16(&Wc[ks * 16 * WN + woff_lo[nb]]);
        const half4_t hi = lds_read_tr16(&Wc[ks * 16 * WN + woff_hi[nb]]);
        return half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    float16_t acc[4][4];   // [column block][token block]
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.f;
    float ss[4] = {0.f, 0.f, 0.f, 0.f};
    // One contraction step = 4 groups (one token block each) of 4 MFMAs.  A wave has its SIMD to itself, so
    // whatever else it issues must sit between MFMAs or the pipe runs dry: every MFMA heads a slot that also
    // carries a piece of the other work -- the sum of squares and gamma multiply of the NEXT group's operand
    // (the next step's first one in the last group), the next step's operand reads (W operands first: its first
    // group needs all four), and, in the second step of a k-tile, a quarter of the stage refill.
    auto step = [&](half8_t& xv, half8_t (&xb)[4], half8_t (&wa)[4], const half8_t& g, half8_t (&xn)[4],
                    half8_t (&wn_)[4], const half_t* Xr, const half_t* Wr, int ks_r, const half8_t& gn,
                    auto&& extra) __attribute__((always_inline)) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            acc[0][mb] = mfma32(wa[0], xv, acc[0][mb]);
            if (mb == 0) wn_[0] = read_w(Wr, ks_r, 0);
            if (mb == 1) wn_[2] = read_w(Wr, ks_r, 2);
            if (mb >= 2) xn[mb] = read_x(Xr, ks_r, mb);
            __builtin_amdgcn_sched_barrier(0);
            acc[1][mb] = mfma32(wa[1], xv, acc[1][mb]);
            const half8_t raw = mb < 3 ? xb[mb + 1] : xn[0];
            if (stats) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const half2_t p = {raw[2 * e], raw[2 * e + 1]};
                    ss[(mb + 1) & 3] = __builtin_amdgcn_fdot2(p, p, ss[(mb + 1) & 3], false);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            acc[2][mb] = mfma32(wa[2], xv, acc[2][mb]);
            const half8_t xv_next = raw * (mb < 3 ? g : gn);
            if (mb == 0) wn_[1] = read_w(Wr, ks_r, 1);
            if (mb == 1) wn_[3] = read_w(Wr, ks_r, 3);
            __builtin_amdgcn_sched_barrier(0);
            acc[3][mb] = mfma32(wa[3], xv, acc[3][mb]);
            if (mb < 2) xn[mb] = read_x(Xr, ks_r, mb);
            extra(mb);
            __builtin_amdgcn_sched_barrier(0);
            xv = xv_next;
        }
    };

    // The k-tile loop runs in whole turns of the 4-stage ring and always fetches ahead: k-tiles past hidden
    // fetch zeros (out-of-range loads) and add nothing, which keeps the loop free of tail branches and the count
    // of loads in flight, on which the waits below rely, the same in every iteration.
    // ---- prologue: all four stages and three gamma slices in flight, then the first operands
    if (use_g) { fetch_g(0, g0); fetch_g(1, g1); fetch_g(2, g2); }
    TRN_FETCH(0, Xs0, Ws0);
    TRN_FETCH(1, Xs1, Ws1);
    TRN_FETCH(2, Xs2, Ws2);
    TRN_FETCH(3, Xs3, Ws3);
    __builtin_amdgcn_s_waitcnt(0x0f70);     // vmcnt(0)
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) { xb0[i] = read_x(Xs0, 0, i); wa0[i] = read_w(Ws0, 0, i); }
    half8_t xv = xb0[0];                    // the operand of the next MFMA group, gamma applied
    if (stats) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const half2_t p = {xv[2 * e], xv[2 * e + 1]};
            ss[0] = __builtin_amdgcn_fdot2(p, p, ss[0], false);
        }
    }
    xv = xv * g0[0];

    // k-tile kt reads stage kt%4: the operands of its first step during the second step of k-tile kt-1, those of
    // its second step during its first.  From the barrier between the two steps on, the stage is free and is
    // refilled with k-tile kt+4 -- three k-tiles before that one's barrier.
    auto ktile = [&](int kt, half_t* Xc, half_t* Wc, const half_t* Xn, const half_t* Wn, const half8_t (&gc)[2],
                     const half8_t (&gn)[2], half8_t (&gf)[2]) __attribute__((always_inline)) {
        step(xv, xb0, wa0, gc[0], xb1, wa1, Xc, Wc, 1, gc[1], [&](int) __attribute__((always_inline)) {});
        // Stage kt+1 must have landed.  Loads complete in issue order, and behind this wave's share of that stage
        // only the refills and gamma slices of the last two k-tiles (2 x (8 + 2) loads) have been issued.
        // lgkmcnt(0): this wave's reads of stage kt have returned, so the refill cannot overtake them.
        if (use_g) __builtin_amdgcn_s_waitcnt(0x4074); else __builtin_amdgcn_s_waitcnt(0x4070);
        // A bare barrier: __syncthreads() would first drain every load in flight, the prefetched stages included.
        // Nothing else needs ordering here -- in this loop LDS is written only by those loads.
        __builtin_amdgcn_s_barrier();       // everyone's share landed; nobody still reads stage kt
        __builtin_amdgcn_sched_barrier(0);
        step(xv, xb1, wa1, gc[1], xb0, wa0, Xn, Wn, 0, gn[0], [&](int i) __attribute__((always_inline)) {
            // gamma three tiles ahead and before the stage loads: its use never has to wait for a stage
            if (i == 0 && use_g) fetch_g(kt + 3, gf);
            TRN_FETCH_ONE(kt + 4, Xc, Wc, i);
        });
    };
    for (int kt = 0; kt < nk; kt += 4) {
        ktile(kt, Xs0, Ws0, Xs1, Ws1, g0, g1, g3);
        ktile(kt + 1, Xs1, Ws1, Xs2, Ws2, g1, g2, g0);
        ktile(kt + 2, Xs2, Ws2, Xs3, Ws3, g2, g3, g1);
        ktile(kt + 3, Xs3, Ws3, Xs0, Ws0, g3, g0, g2);
    }
#undef TRN_FETCH_ONE
#undef TRN_FETCH

    // row rstd from the first column group's sums: a lane holds the columns 8h..8h+7 of each 16 of its tokens
    if (stats) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            const float s = half_sum(ss[mb]);
            if (h == 0) rstd_s[wm * 128 + mb * 32 + c] = 1.0f / __builtin_sqrtf(s / (float)a.K + a.eps);
        }
    }
    __syncthreads();                        // also: every wave is done with the stages

    // ---- epilogue: scale, transpose 64 tokens x 64 columns at a time through LDS (two stage arrays of 16 KB
    // per wave, used alternately), store 16 bytes per lane: 8 lanes cover the 64 columns of a token, 8 tokens per
    // store instruction
    {
        constexpr int OP = 64 + 4;                          // pitch in halfs; 64*68*2 = 8704 bytes <= a stage
        half_t* ot = wave == 0 ? Xs0 : wave == 1 ? Xs1 : wave == 2 ? Xs2 : Xs3;
        const int orow = lane >> 3, ocol = (lane & 7) * 8;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            float r[2];
#pragma unroll
            for (int ml = 0; ml < 2; ++ml) r[ml] = a.norm ? rstd_s[wm * 128 + (2 * p + ml) * 32 + c] : 1.0f;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
#pragma unroll
                for (int ml = 0; ml < 2; ++ml)
#pragma unroll
                    for (int nl = 0; nl < 2; ++nl)
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4) {
                            half4_t ov;
#pragma unroll
                            for (int e = 0; e < 4; ++e) ov[e] = (half_t)(acc[2 * q + nl][2 * p + ml][r4 * 4 + e] * r[ml]);
                            *reinterpret_cast<half4_t*>(&ot[(ml * 32 + c) * OP + nl * 32 + 8 * r4 + 4 * h]) = ov;
                        }
                // (LDS operations of one wave execute in order: its reads below see its writes above, and the
                // next pass's writes come after these reads)
                const int n = n0 + wn * 128 + q * 64 + ocol;
                half_t* obase = P.out + (int64_t)(n / a.head_dim) * P.stride_h + (n % a.head_dim);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int tl = j * 8 + orow, t = m0 + wm * 128 + p * 64 + tl;
                    const uint2_t lo = *reinterpret_cast<const uint2_t*>(&ot[tl * OP + ocol]);
                    const uint2_t hi = *reinterpret_cast<const uint2_t*>(&ot[tl * OP + ocol + 4]);
                    if (t < a.T && n < P.n)
                        *reinterpret_cast<uint4_t*>(obase + (int64_t)t * P.stride_s) = uint4_t{lo.x, lo.y, hi.x, hi.y};
                }
            }
        }
    }
#endif
}

int launch_prenorm_qkv_wide(GemmArgs a, int64_t n_q, int64_t n_kv, hipStream_t stream) {
    a.n_mtiles = (a.T + WM - 1) / WM;
    const int tq = (int)((n_q + WN - 1) / WN), tkv = (int)((n_kv + WN - 1) / WN);
    a.p[0].tile0 = 0; a.p[1].tile0 = tq; a.p[2].tile0 = tq + tkv;
    a.n_panels = tq + 2 * tkv;
    a.panels_per_xcd = (a.n_panels + 7) / 8;
    const int64_t grid = (int64_t)8 * a.panels_per_xcd * a.n_mtiles;
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    hipLaunchKernelGGL(prenorm_qkv_wide_kernel, dim3((unsigned)grid), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}

// Workgroups the wide tiling would launch (useful ones, not counting the padding of the XCD mapping).
int64_t prenorm_qkv_wide_tiles(int64_t tokens, int64_t n_q, int64_t n_kv) {
    return ((tokens + WM - 1) / WM) * ((n_q + WN - 1) / WN + 2 * ((n_kv + WN - 1) / WN));
}

}  // namespace trn
