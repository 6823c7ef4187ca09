// Fused RMSNorm + Q/K/V projection GEMM, 256-token x 256- or 192-column workgroup tiles (large problems).
//
// Same arithmetic and MFMA mapping as the 128 x 128 kernel (C^T = W^T X^T with 32x32x16 fp16 MFMAs, a lane owns
// one token), re-balanced for what limits a large GEMM on this chip:
//   * 4 waves, one per SIMD, each a 128-token x 128-column sub-tile (4 x 4 MFMA blocks, 256 accumulator
//     registers -- the whole AGPR file of a wave that has its SIMD to itself): every 16-byte LDS operand feeds
//     four MFMAs instead of two, so LDS bytes and LDS instructions per MFMA are halved.  With NB = 3 the sub-tile
//     is 128 x 96 and the workgroup tile 256 x 192: three quarters of the work per tile, for problems whose
//     256-wide tiles would fill only three quarters of the chip (2048 tokens x 6144 columns: 192 tiles on 256 CUs).
//   * The columns of Q, K and V form one axis of 64-column groups (each output padded to whole groups); a tile is
//     NB consecutive groups and may straddle two outputs: every group has its own buffer descriptor, and every
//     32-column block of the epilogue its own output.
//   * Both operands go straight from global memory into LDS (buffer_load ... lds, XOR-swizzled rows); no
//     register staging and no LDS writes from the VALU.  gamma is multiplied into the W operand after it is read
//     back from LDS (one packed fp16 multiply per pair: the correctly rounded product; a lane's W^T operand holds the
//     same eight contraction columns as its X^T operand, and a step has NB W operands against four X operands), and
//     the waves of the first column group sum the squares of X with the fp32 dot-product instruction for the row rstd.
//   * Four stages of 32 contraction columns: a stage is requested three k-tiles before its first use,
//     which at 256 x 256 flops per staged column covers the L2 / HBM latency.
//   * The one barrier per k-tile sits between the two 16-column halves of the tile's MFMAs, after the second
//     half's operands are already in registers: waves reach it with MFMAs in flight, and the first operands of
//     the next tile are read right behind it, so neither the barrier nor the LDS latency drains the MFMA pipe.
#include "prenorm_qkv.h"

namespace trn {

[[maybe_unused]] constexpr int WM = 256, WK = 32, WG = 64;       // tokens per tile, contraction columns per stage, columns per group

// Chunk swizzle of a W group row (eight 16-byte chunks, 128 bytes: consecutive rows alternate between the two
// halves of the 64 banks): with bit 2 from row bit 1 and the low bits from row bits 2-3, the four consecutive rows
// x four consecutive chunks of one phase of the transposing read touch every bank once.
__device__ __forceinline__ int gswz(int r) { return (((r >> 1) & 1) << 2) | ((r >> 2) & 3); }

// G: gamma is multiplied into the W operand (norm on and a gamma given); without it the multiply, the gamma
// loads and their ring leave the loop.
template <int NB, bool G>
__global__ __launch_bounds__(256, 1) void prenorm_qkv_wide_kernel(const GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    // One array per stage and operand: the compiler orders LDS reads after outstanding global->LDS loads that may
    // alias them, and only distinct variables are provably disjoint.
    __shared__ __attribute__((aligned(1024))) half_t Xs0[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs1[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs2[WM * WK];
    __shared__ __attribute__((aligned(1024))) half_t Xs3[WM * WK];
    constexpr int WN = NB * WG;                        // columns per tile; a W stage is NB groups of [32 rows][64 columns]
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
    const int g_first = nt_all * NB, m0 = mt * WM;      // first column group of the tile
    const int nk = (a.K + WK - 1) / WK;
    constexpr int kOut = 0x7ffffff0;                  // a byte offset past every buffer: the load returns zeros

    // ---- W stage: per group 32 rows x 128 bytes.  A wave-wide load covers 8 rows of one group; this wave loads rows
    // 8*wave + lane/8 of every group.  A group belongs to one output: its own descriptor, column offset and pitch.
    // (Columns of a ragged last group past the output's width read the next row or zeros; they are never stored.)
    __amdgpu_buffer_rsrc_t wrs[NB];
    int w_vo[NB], w_tile[NB];
#pragma unroll
    for (int g = 0; g < NB; ++g) {
        const int gg = g_first + g;
        const int pi = gg >= a.p[2].tile0 ? 2 : (gg >= a.p[1].tile0 ? 1 : 0);
        const half_t* w = pi == 2 ? a.p[2].w : pi == 1 ? a.p[1].w : a.p[0].w;
        const int64_t ldw = pi == 2 ? a.p[2].ldw : pi == 1 ? a.p[1].ldw : a.p[0].ldw;
        const int n = pi == 2 ? a.p[2].n : pi == 1 ? a.p[1].n : a.p[0].n;
        const int t0 = pi == 2 ? a.p[2].tile0 : pi == 1 ? a.p[1].tile0 : 0;
        wrs[g] = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, (int)(((int64_t)(a.K - 1) * ldw + n) * 2), 0x00020000);
        const int r = 8 * wave + (lane >> 3);
        w_vo[g] = (int)(r * ldw * 2) + ((gg - t0) * WG + 8 * ((lane & 7) ^ gswz(r))) * 2;
        w_tile[g] = (int)(WK * ldw * 2);
    }
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
    // load pair i_ (one X wave-wide load and, for i_ < NB, the W load of group i_) of stage kt_; columns past
    // hidden hold the next row's data in X: read zeros instead; W rows past hidden are out of range by themselves
#define TRN_FETCH_ONE(kt_, xd_, wd_, i_)                                                                         \
    do {                                                                                                         \
        const bool drop_ = (kt_) * WK + 8 * x_chunk >= a.K;                                                      \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                                \
            xrs, (__attribute__((address_space(3))) void*)(&xd_[(64 * (i_) + 16 * wave) * WK]), 16,              \
            drop_ ? kOut : x_vo[i_], (kt_) * WK * 2, 0, 0);                                                      \
        if ((i_) < NB)                                                                                           \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
                wrs[(i_) < NB ? (i_) : 0], (__attribute__((address_space(3))) void*)(&wd_[((i_) * WK + 8 * wave) * WG]), 16, \
                w_vo[(i_) < NB ? (i_) : 0], (kt_) * w_tile[(i_) < NB ? (i_) : 0], 0, 0);                         \
    } while (0)
#define TRN_FETCH(kt_, xd_, wd_) _Pragma("unroll") for (int fi_ = 0; fi_ < 4; ++fi_) TRN_FETCH_ONE(kt_, xd_, wd_, fi_)

    // ---- gamma: the operands of contraction step ks hold columns kt*32 + ks*16 + 8h .. +7 (of the lane's token in
    // X^T, of the lane's output column in W^T).
    constexpr bool use_g = G;
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
    // (wn*NB + nb)*32 + 16*((lane/16)%2) + 4*(lane%4) of the tile, i.e. group (wn*NB + nb)/2, chunks 4*((wn*NB + nb)%2) ..
    int woff_lo[NB], woff_hi[NB];
    {
        const int rl = 8 * h + ((lane & 15) >> 2), rh = rl + 4;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int blk = wn * NB + nb, chunk = 4 * (blk & 1) + lc;
            woff_lo[nb] = (blk >> 1) * WK * WG + rl * WG + ((chunk ^ gswz(rl)) << 3) + sub;
            woff_hi[nb] = (blk >> 1) * WK * WG + rh * WG + ((chunk ^ gswz(rh)) << 3) + sub;
        }
    }
    half8_t xb0[4], xb1[4], wa0[NB], wa1[NB];           // operands of the two contraction steps of a k-tile
    auto read_x = [&](const half_t* Xc, int ks, int mb) __attribute__((always_inline)) {
        return *reinterpret_cast<const half8_t*>(&Xc[xoff[ks] + mb * 32 * WK]);
    };
    auto read_w = [&](const half_t* Wc, int ks, int nb) __attribute__((always_inline)) {
        const half4_t lo = lds_read_tr16(&Wc[ks * 16 * WG + woff_lo[nb]]);
        const half4_t hi = lds_read_tr16(&Wc[ks * 16 * WG + woff_hi[nb]]);
        return half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    float16_t acc[NB][4];   // [column block][token block]
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.f;
    float ss[4] = {0.f, 0.f, 0.f, 0.f};
    // One contraction step = 4 groups (one token block each) of NB MFMAs.  A wave has its SIMD to itself, so
    // whatever else it issues must sit between MFMAs or the pipe runs dry: every MFMA heads a slot that also
    // carries a piece of the other work -- the sum of squares of the NEXT group's X operand (the next step's first
    // one in the last group), the next step's operand reads (W operands first: its first group needs all of them),
    // the gamma multiply of those W operands in the last group (by then they have arrived), and, in the second step
    // of a k-tile, a quarter of the stage refill.
    auto step = [&](half8_t& xv, half8_t (&xb)[4], half8_t (&wa)[NB], const half8_t& g, half8_t (&xn)[4],
                    half8_t (&wn_)[NB], const half_t* Xr, const half_t* Wr, int ks_r, const half8_t& gn,
                    auto&& extra) __attribute__((always_inline)) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            // (the column blocks are walked forwards for even token blocks and backwards for odd ones, so that from one MFMA
            // to the next only one of the two operands changes: 0.5 % of the kernel's time at the board's power limit)
            { constexpr int z = 0; const int nbx = (mb & 1) ? NB - 1 - z : z; acc[nbx][mb] = mfma32(wa[nbx], xv, acc[nbx][mb]); }
            if (mb == 0) wn_[0] = read_w(Wr, ks_r, 0);
            if (mb == 1) wn_[2] = read_w(Wr, ks_r, 2);
            if (mb >= 2) xn[mb] = read_x(Xr, ks_r, mb);
            __builtin_amdgcn_sched_barrier(0);
            { constexpr int z = 1; const int nbx = (mb & 1) ? NB - 1 - z : z; acc[nbx][mb] = mfma32(wa[nbx], xv, acc[nbx][mb]); }
            const half8_t raw = mb < 3 ? xb[mb + 1] : xn[0];
            if (stats) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const half2_t p = {raw[2 * e], raw[2 * e + 1]};
                    ss[(mb + 1) & 3] = __builtin_amdgcn_fdot2(p, p, ss[(mb + 1) & 3], false);
                }
            }
            if constexpr (NB == 3) {
                if (mb == 0) wn_[1] = read_w(Wr, ks_r, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            { constexpr int z = 2; const int nbx = (mb & 1) ? NB - 1 - z : z; acc[nbx][mb] = mfma32(wa[nbx], xv, acc[nbx][mb]); }
            const half8_t xv_next = raw;
            if constexpr (NB == 4) {
                if (mb == 0) wn_[1] = read_w(Wr, ks_r, 1);
                if (mb == 1) wn_[3] = read_w(Wr, ks_r, 3);
                __builtin_amdgcn_sched_barrier(0);
                { constexpr int z = 3; const int nbx = (mb & 1) ? NB - 1 - z : z; acc[nbx][mb] = mfma32(wa[nbx], xv, acc[nbx][mb]); }
            }
            if (mb < 2) xn[mb] = read_x(Xr, ks_r, mb);
            if constexpr (G) {
                if (mb == 3) {
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) wn_[nb] = wn_[nb] * gn;
                }
            }
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
    for (int i = 0; i < 4; ++i) xb0[i] = read_x(Xs0, 0, i);
#pragma unroll
    for (int i = 0; i < NB; ++i) wa0[i] = read_w(Ws0, 0, i);
    half8_t xv = xb0[0];                    // the X operand of the next MFMA group
    if (stats) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const half2_t p = {xv[2 * e], xv[2 * e + 1]};
            ss[0] = __builtin_amdgcn_fdot2(p, p, ss[0], false);
        }
    }
    if (G) {
#pragma unroll
        for (int i = 0; i < NB; ++i) wa0[i] = wa0[i] * g0[0];
    }

    // k-tile kt reads stage kt%4: the operands of its first step during the second step of k-tile kt-1, those of
    // its second step during its first.  From the barrier between the two steps on, the stage is free and is
    // refilled with k-tile kt+4 -- three k-tiles before that one's barrier.
    auto ktile = [&](int kt, half_t* Xc, half_t* Wc, const half_t* Xn, const half_t* Wn, const half8_t (&gc)[2],
                     const half8_t (&gn)[2], half8_t (&gf)[2]) __attribute__((always_inline)) {
        step(xv, xb0, wa0, gc[0], xb1, wa1, Xc, Wc, 1, gc[1], [&](int) __attribute__((always_inline)) {});
        // Stage kt+1 must have landed.  Loads complete in issue order, and behind this wave's share of that stage
        // only the refills and gamma slices of the last two k-tiles (2 x (4 + NB + 2) loads) have been issued.
        // lgkmcnt(0): this wave's reads of stage kt have returned, so the refill cannot overtake them.
        constexpr int kBehindG = 2 * (4 + NB + 2), kBehind = 2 * (4 + NB);
        if (use_g) __builtin_amdgcn_s_waitcnt(0x0070 | (kBehindG & 15) | ((kBehindG >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0070 | (kBehind & 15) | ((kBehind >> 4) << 14));
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

    // ---- epilogue: scale, transpose 64 tokens x 32 columns at a time through LDS (this wave's own X stage),
    // store 16 bytes per lane: 4 lanes cover the 32 columns of a token, 16 tokens per store instruction.  A
    // 32-column block lies in one group, hence in one output and (head_dim being a multiple of 32) in one head.
    {
        constexpr int OP = 32 + 8;                          // pitch in halfs
        half_t* ot = wave == 0 ? Xs0 : wave == 1 ? Xs1 : wave == 2 ? Xs2 : Xs3;
        const int orow = lane >> 2, ocol = (lane & 3) * 8;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int blk = wn * NB + nb, gg = g_first + (blk >> 1);
            const int pi = gg >= a.p[2].tile0 ? 2 : (gg >= a.p[1].tile0 ? 1 : 0);
            half_t* out = pi == 2 ? a.p[2].out : pi == 1 ? a.p[1].out : a.p[0].out;
            const int64_t stride_h = pi == 2 ? a.p[2].stride_h : pi == 1 ? a.p[1].stride_h : a.p[0].stride_h;
            const int64_t stride_s = pi == 2 ? a.p[2].stride_s : pi == 1 ? a.p[1].stride_s : a.p[0].stride_s;
            const int pn = pi == 2 ? a.p[2].n : pi == 1 ? a.p[1].n : a.p[0].n;
            const int t0 = pi == 2 ? a.p[2].tile0 : pi == 1 ? a.p[1].tile0 : 0;
            const half_t* addend = pi == 2 ? a.p[2].addend : pi == 1 ? a.p[1].addend : a.p[0].addend;
            const int n = (gg - t0) * WG + (blk & 1) * 32 + ocol;
            const int64_t o_off = (int64_t)(n / a.head_dim) * stride_h + (n % a.head_dim);
            half_t* obase = out + o_off;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
#pragma unroll
                for (int ml = 0; ml < 2; ++ml) {
                    const float r = a.norm ? rstd_s[wm * 128 + (2 * p + ml) * 32 + c] : 1.0f;
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        half4_t ov;
#pragma unroll
                        for (int e = 0; e < 4; ++e) ov[e] = (half_t)(acc[nb][2 * p + ml][r4 * 4 + e] * r);
                        *reinterpret_cast<half4_t*>(&ot[(ml * 32 + c) * OP + 8 * r4 + 4 * h]) = ov;
                    }
                }
                // (LDS operations of one wave execute in order: its reads below see its writes above, and the
                // next pass's writes come after these reads)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int tl = j * 16 + orow, t = m0 + wm * 128 + p * 64 + tl;
                    half8_t ov = *reinterpret_cast<const half8_t*>(&ot[tl * OP + ocol]);
                    if (t < a.T && n < pn) {
                        if (addend) {
                            const half8_t ad = *reinterpret_cast<const half8_t*>(addend + o_off + (int64_t)t * stride_s);
#pragma unroll
                            for (int e = 0; e < 8; ++e) ov[e] = (half_t)((float)ov[e] + (float)ad[e]);
                        }
                        *reinterpret_cast<half8_t*>(obase + (int64_t)t * stride_s) = ov;
                    }
                }
            }
        }
    }
#endif
}

// Tiles of nb 64-column groups over the group axis [Q | K | V], each output padded to whole groups.
static int64_t wide_tiles(const GemmArgs& a, int nb) {
    int64_t groups = 0;
    for (int i = 0; i < 3; ++i) groups += (a.p[i].n + WG - 1) / WG;
    return (((int64_t)a.T + WM - 1) / WM) * ((groups + nb - 1) / nb);
}

// 192-column tiles when they keep the chip busier: the time is (rounds of 256 workgroups) x (work per tile), and a
// 192-wide tile does 3/4 of the work of a 256-wide one at slightly lower efficiency (fewer MFMAs per operand read).
static bool narrow_is_better(const GemmArgs& a) {
    const int64_t r4 = (wide_tiles(a, 4) + 255) / 256, r3 = (wide_tiles(a, 3) + 255) / 256;
    return r3 * 3 * 100 < r4 * 4 * 95;
}

int launch_prenorm_qkv_wide(GemmArgs a, hipStream_t stream) {
    const int nb = narrow_is_better(a) ? 3 : 4;
    a.n_mtiles = (a.T + WM - 1) / WM;
    int g0 = 0;
    for (int i = 0; i < 3; ++i) { a.p[i].tile0 = g0; g0 += (a.p[i].n + WG - 1) / WG; }      // first group of each output
    a.n_panels = (g0 + nb - 1) / nb;
    a.panels_per_xcd = (a.n_panels + 7) / 8;
    const int64_t grid = (int64_t)8 * a.panels_per_xcd * a.n_mtiles;
    if (grid > 0x7fffffffLL) return TRN_E_SHAPE;
    const bool g = a.gamma != nullptr && a.norm;
    auto* kernel = nb == 3 ? (g ? prenorm_qkv_wide_kernel<3, true> : prenorm_qkv_wide_kernel<3, false>)
                           : (g ? prenorm_qkv_wide_kernel<4, true> : prenorm_qkv_wide_kernel<4, false>);
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}

// Workgroups the 256-column tiling would launch (useful ones, not counting the padding of the XCD mapping).
int64_t prenorm_qkv_wide_tiles(const GemmArgs& a) { return wide_tiles(a, 4); }

}  // namespace trn
