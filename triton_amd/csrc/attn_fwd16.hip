// Flash attention forward for gfx950 on the 16x16x32 MFMA: O = softmax(scale * Q K^T [+causal]) V, GQA/MQA,
// head_dim 64/128, no score perturbation (that variant stays on the 32x32x16 kernel in attn_fwd.hip).
//
// Why a second kernel for the same arithmetic: at these shapes the chip is power-limited, and per flop the
// 16x16x32 instruction reads and writes half as many accumulator registers as the 32x32x16 one (a 16x16 fp32 block
// per 16 K flop against a 32x32 block per 32 K flop).  Issued back to back on random operands it sustains about
// 17 % more flops at the board's power limit; whatever part of that survives the softmax work is free.
//
// Formulation (transposed, as in attn_fwd.hip).  A wave owns 32 queries as two blocks of 16 (qb); lane l = 16 g + n
// holds queries 16 qb + n.  Per 32-key block, split in two halves of 16 keys (kb):
//     S^T(kb, qb)[key][query] = K[16 kb + key][:] . Q[16 qb + query][:]   A = K rows from LDS (one 16-byte read:
//                               row n, contraction columns 32 ks + 8 g ..+7), B = Q^T in registers
//   the lane receives keys 16 kb + 4 g + 0..3 of its two queries: 8 keys per query, the other 24 sit in the
//   lanes n + 16, n + 32, n + 48.  The running max is kept equal in the four lanes of a query, and whether it must
//   rise is decided from the lane's own 8 keys (any lane of the wave over the threshold raises it for all), so the
//   common path has no cross-lane traffic at all.  Row sums come from the matrix pipe (an all-ones A operand).
//     O^T(db, qb)[d][query] += V^T[16 db + d][slot] * P^T[slot][query]   one MFMA per 32-key block (K = 32)
//   contraction slot 8 g + j of a lane is key 4 g + j (j < 4) or 16 + 4 g + (j - 4): exactly the keys whose
//   scores the lane holds, so P goes from the S^T accumulators to the B operand without leaving the lane, and the
//   A operand takes its two transposing reads from rows 4 g .. and 16 + 4 g .. of the V stage.
// The exponent comes out of the matrix pipe ready-made: Q is multiplied by scale * log2(e) once in the prologue, and
// every score chain starts from the accumulator {-m} instead of zero, so S^T arrives as s - m and the softmax costs
// one v_exp_f32 per score and nothing else (the multiply-subtract it replaces was a quarter of the loop's vector
// instructions).  When the lazy maximum rises, the scores already in flight are shifted along with it.
// Staging (global -> LDS loads, XOR swizzle, two stages each for K and V, one barrier per 64-key tile), the grid
// and the lazy running maximum are those of attn_fwd.hip.
#include "attn.h"
#include <type_traits>

namespace trn {

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// v_permlane16_swap exchanges the odd 16-lane rows of one register with the even rows of another: from two
// copies of x it leaves the values of rows {0, 0, 2, 2} and {1, 1, 3, 3}.  Followed by the 32-lane exchange this
// combines the four lanes n, n + 16, n + 32, n + 48.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ int imax3(int a, int b, int c) { return max(max(a, b), c); }
__device__ __forceinline__ float quad_max(float x) { float a = x, b = x; swap_rows16(a, b); return half_max(fmaxf(a, b)); }
__device__ __forceinline__ float quad_sum(float x) { float a = x, b = x; swap_rows16(a, b); return half_sum(a + b); }

// XOR swizzle of the 16-byte chunk index within a stage row for this kernel's access patterns.  The LDS has 64
// banks (256 bytes per clock).  A 16-byte read is served 16 lanes at a time, and the lanes served together are
// {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same plus 32 (measured: two lanes that read different addresses
// in the same bank cost a cycle exactly when both are in one of these sets); the transposing 8-byte read is served
// in halves of the wave.  (a) A K operand read has lane 16 g + n on row n at logical chunk 4 ks + g, so a set holds
// the rows {0-3, 12-15} at one chunk and the rows {4-11} at its neighbour: no two rows, one from each, may have
// swizzles that differ in bit 0 only.  (b) A transposing V read has each half of the wave on 8 consecutive rows x 2
// adjacent chunks: the swizzle without bit 0 must be distinct over those rows.  (Rows of 128 bytes: two share a
// 256-byte line, and the conditions hold per row parity.)
template <int D> __device__ __forceinline__ int swz16(int r) {
    if constexpr (D == 128) return ((r & 7) << 1) ^ ((r & 8) ? 9 : 0);       // rows 12 apart differ in bit 0 only
    else return r & 6;
}

struct Scores16 { float4_t s[2][2]; };      // [key half][query block]

template <int D, int NW, bool PAIRED>
__global__ __launch_bounds__(NW * 64, NW == 8 ? 1 : 2) void attn_fwd16_kernel(const AttnArgs a) {
    static_assert(!PAIRED || NW == 8, "paired query tiles are two groups of four waves");
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BN = 64;       // keys per LDS stage (two 32-key blocks)
    constexpr int NS = D / 8;    // MFMA slots per phase: 2 key halves x 2 query blocks x D/32 steps of S^T; D/16 x 2 of P V
    constexpr int NKS = D / 32;  // contraction steps of S^T
    constexpr int NOP = D / 16;  // LDS operands per phase (each feeds the MFMAs of both query blocks)
    constexpr int CPR = D / 8;   // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;            // stage rows covered by one wave-wide 1 KB load
    constexpr int NI = BN / (RPI * NW);      // such loads per wave per stage (K and V each)
    constexpr int BM = 32 * NW;              // queries per workgroup
    __shared__ __attribute__((aligned(1024))) half_t Ks0[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Ks1[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Vs0[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Vs1[BN * D];

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const int BH = a.B * a.Hq;
    const int j = blockIdx.x % BH;
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;

    const int off = a.Skv - a.Sq;                       // causal: query i sees keys <= i + off
    // Query rows.  Plain mode: the workgroup owns BM consecutive queries, latest (heaviest under a causal mask) tiles
    // first.  Paired mode (NW = 8, causal, a grid too small for a second round to even out the tiles' lengths): waves
    // 0-3 own the 128-query tile h, waves 4-7 the tile n - 1 - h from the other end, so that every workgroup has the
    // same amount of work and each SIMD holds one long and one short wave.  K/V staging follows the later tile; the
    // early waves stop at their own last visible tile as they do in plain mode.
    int q0, q_last, wq0;
    bool idle = false;
    if constexpr (PAIRED) {
        const int lt = (int)(blockIdx.x / BH), ht = a.n_qtiles - 1 - lt;     // n_qtiles counts 128-query tiles here
        q0 = ht * 128; q_last = q0 + 127;
        idle = wave >= 4 && lt == ht;                                       // odd tile count: the middle one is alone
        wq0 = (wave < 4 ? ht : lt) * 128 + (wave & 3) * 32;
        if (idle) wq0 = a.Sq;                                               // loads clamp, stores are predicated off
    } else {
        q0 = (a.n_qtiles - 1 - (int)(blockIdx.x / BH)) * BM; q_last = q0 + BM - 1;
        wq0 = q0 + wave * 32;                           // first query of this wave
    }
    int qrow[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) qrow[qb] = wq0 + 16 * qb + n;
    half8_t qB[2][NKS];

    // ---- LDS read offsets (halfs).  K operand (ks, kb): row 16 kb + n of a 32-key block, logical chunk 4 ks + g4
    // (the swizzle depends on the row's low four bits only, so the second key half is a constant 16 rows further).
    int koff[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) koff[ks] = n * D + (((4 * ks + g4) ^ swz16<D>(n)) << 3);
    // V^T operand db through the transposing read: in each 16-lane group lanes 4r..4r+3 supply stage row r; this
    // lane's piece is row 4 g4 + n/4 (second read: 16 rows further), head_dim columns 16 db + 4 (n%4) ..+3.
    int voff[NOP];
    {
        const int rl = 4 * g4 + (n >> 2), lc = (n & 3) >> 1, sub = (n & 1) * 4;
#pragma unroll
        for (int db = 0; db < NOP; ++db) voff[db] = rl * D + (((2 * db + lc) ^ swz16<D>(rl)) << 3) + sub;
    }

    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    float4_t oacc[NOP][2];                  // [16 head_dim columns][query block]
#pragma unroll
    for (int i = 0; i < NOP; ++i) oacc[i][0] = oacc[i][1] = zero;
    float m[2] = {-INFINITY, -INFINITY};    // reference max (log2 domain), equal in the four lanes of a query
    float4_t negm[2];                       // {-m} x 4: the initial accumulator of every score chain, so that the
                                            // scores arrive as s - m and the exponential needs no subtraction
    // Row sums come out of the matrix pipe as well: one more MFMA per query block whose A operand is all ones leaves
    // the sum of the block's (fp16-rounded) probabilities of each query in every row of a 16 x 16 accumulator.  Two
    // MFMAs per 32-key block instead of eight dot-product instructions, each of which costs two VALU issue slots.
    float4_t lacc[2] = {zero, zero};

    int ntiles = (a.Skv + BN - 1) / BN;
    if (a.causal) ntiles = min(ntiles, (min(q_last, a.Sq - 1) + off) / BN + 1);

    // ---- staging: direct global -> LDS loads; keys past the end read as zeros
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.k + b * a.kb + kvh * a.kh), 0, (int)(((int64_t)(a.Skv - 1) * a.ks + D) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.v + b * a.vb + kvh * a.vh), 0, (int)(((int64_t)(a.Skv - 1) * a.vs + D) * 2), 0x00020000);
    const int st_row = wave * RPI + lane / CPR;
    const int st_chunk = (lane % CPR) ^ swz16<D>(st_row);
    const int kvo = (int)(st_row * a.ks * 2) + st_chunk * 16;
    const int vvo = (int)(st_row * a.vs * 2) + st_chunk * 16;
    const int krow_bytes = (int)(RPI * a.ks * 2), vrow_bytes = (int)(RPI * a.vs * 2);
    const int ktile_bytes = (int)(BN * a.ks * 2), vtile_bytes = (int)(BN * a.vs * 2);
#define TRN_FETCH_K(jt_, dst_) fetch_tile<NI, D, NW>(krs, &dst_[wave * RPI * D], kvo, (jt_) * ktile_bytes, krow_bytes)
#define TRN_FETCH_V(jt_, dst_) fetch_tile<NI, D, NW>(vrs, &dst_[wave * RPI * D], vvo, (jt_) * vtile_bytes, vrow_bytes)

    const int wb = wq0 + off;          // key index bound of this wave's first query
    auto needs_mask = [&](int key0) { return (key0 + 32 > a.Skv) || (a.causal && key0 + 31 > wb); };

    // Scores of a 32-key block starting at key0, just produced: keys past the end and, under a causal mask, keys
    // after the query become -inf.
    auto mask_block = [&](Scores16& sx, int key0) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = key0 + 16 * kb + 4 * g4 + i;
                    const bool ok = key < a.Skv && (!a.causal || key <= qrow[qb] + off);
                    sx.s[kb][qb][i] = ok ? sx.s[kb][qb][i] : -INFINITY;
                }
    };
    // The lane's maximum per query over its 8 keys of the block.
    auto block_max = [&](const Scores16& sx, float (&smax)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float4_t& u = sx.s[0][qb];
            const float4_t& w = sx.s[1][qb];
            smax[qb] = fmaxf(max3(u[0], u[1], u[2]), max3(u[3], w[0], w[1]));
            smax[qb] = max3(smax[qb], w[2], w[3]);
        }
    };
    // Is a rescale due?  The reference m is lazy (raised only when some score exceeds it by more than 2^8: see
    // attn_fwd.hip), the scores arrive relative to it, and the decision is wave-uniform, so only whether any of the
    // lane's 16 scores exceeds 8 matters.  For that the bit patterns will do: non-negative floats order as signed
    // integers and every negative float (masked scores included) lies below them.  One three-way integer maximum per
    // two scores, both queries of the lane together, no canonicalising of the operands (9 vector instructions per block
    // against 15 for two float maxima); the per-query maxima are formed on the rare path only.  In four pieces, one per
    // accumulator quad, so that they sit behind four different MFMAs.
    auto max_piece = [&](const Scores16& sx, int piece, int mx) __attribute__((always_inline)) {
        const float4_t& u = sx.s[piece >> 1][piece & 1];
        if (piece == 0) return max(imax3(__float_as_int(u[0]), __float_as_int(u[1]), __float_as_int(u[2])), __float_as_int(u[3]));
        mx = imax3(mx, __float_as_int(u[0]), __float_as_int(u[1]));
        return imax3(mx, __float_as_int(u[2]), __float_as_int(u[3]));
    };
    // the scores sx already in flight are relative to m: they move with it
    auto rescale = [&](Scores16& sx) __attribute__((always_inline)) {
        float smax[2];
        block_max(sx, smax);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            const float up = fmaxf(0.f, quad_max(smax[qb]));
            const float alpha = fast_exp2(-up);
            sx.s[0][qb] = sx.s[0][qb] - up;
            sx.s[1][qb] = sx.s[1][qb] - up;
            negm[qb] = negm[qb] - up;                   // (in place, like the accumulators: a fresh vector here makes
                                                        // the path that skips the rescale copy it every block)
            lacc[qb] = lacc[qb] * alpha;
#pragma unroll
            for (int i = 0; i < NOP; ++i)
                oacc[i][qb] = oacc[i][qb] * alpha;      // (as one vector operation: written per element, the path that
                                                        // skips the rescale ends up copying every accumulator)
            m[qb] = m[qb] + up;
        }
    };

    const half_t one = (half_t)1.f;
    const half8_t ones8 = {one, one, one, one, one, one, one, one};
    constexpr int NQ = 2;   // operand look-ahead, in operands (= 2 NQ MFMA slots; 4 measured no better, twice)
    static_assert(NOP % NQ == 0, "the operand window must divide the operands of a phase");
    half8_t ka[NQ];    // K operands of the next block's S^T, a rolling window ahead of use
    half8_t va[NQ];    // V^T operands of this block's P V, likewise
    auto load_k = [&](const half_t* Kb, int op, int reg) __attribute__((always_inline)) {       // op = 2 ks + kb
        ka[reg] = *reinterpret_cast<const half8_t*>(&Kb[(op & 1) * 16 * D + koff[op >> 1]]);
    };

    // One pipeline step for block B whose scores sc are complete, masked and reflected in m:
    //   phase A: MFMA: S^T of block B+1                  | VALU: P = exp2(sc*c1 - m), fp16, row sums
    //   phase B: MFMA: O^T += V^T P^T                    | VALU: mask + max of block B+1's scores
    // Every LDS operand feeds two consecutive MFMAs (the two query blocks); it is requested NQ operands before its
    // first use, into the register its predecessor has just vacated.  With SYNC (first block of a 64-key tile) the
    // tile hand-over sits right after the last request to the tile's own K stage.
    // MAYMASK = false: the caller knows that block B+1 needs no mask, and the test and its branch (which would sit in
    // the middle of phase B and split the slot sequence) are not compiled in.
    auto step = [&](bool masked_next, auto maymask_tag, auto sync_tag, Scores16& sc, Scores16& sn, const half_t* Vblk, const half_t* K1,
                    const half_t* K2, int key0_next, auto&& handover) __attribute__((always_inline)) {
        constexpr bool SYNC = decltype(sync_tag)::value;
        constexpr bool MAYMASK = decltype(maymask_tag)::value;
        half8_t pB[2];
        auto load_v = [&](int db, int reg) __attribute__((always_inline)) {
            const half4_t lo = lds_read_tr16(Vblk + voff[db]);              // keys 4 g4 .. +3, dim 16 db + n
            const half4_t hi = lds_read_tr16(Vblk + 16 * D + voff[db]);     // keys 16 + 4 g4 .. +3
            va[reg] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        auto exp_pair = [&](int p) __attribute__((always_inline)) {        // scores 2 (p%2), +1 of key half (p/2)%2, query block p/4
            const int qb = p >> 2, kb = (p >> 1) & 1, i0 = 2 * (p & 1);
            const float p0 = fast_exp2(sc.s[kb][qb][i0]);
            const float p1 = fast_exp2(sc.s[kb][qb][i0 + 1]);
            uint32_t u = pack_half2(p0, p1);
            asm volatile("" : "+v"(u));     // keeps the pair's work in this slot (it is otherwise sunk past the hand-over)
            const half2_t pp = __builtin_bit_cast(half2_t, u);
            pB[qb][4 * kb + i0] = pp[0]; pB[qb][4 * kb + i0 + 1] = pp[1];
        };
        // ---- phase A ----
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            // (Gray order over the operand pair: from one MFMA to the next either the LDS operand or the query block
            // changes, never both -- 0.7 % of the kernel's time on N(0,1) data, where the time is the board's power)
            const int op = i >> 1, ks = op >> 1, kb = op & 1, qb = (i & 1) ^ (op & 1);
            if constexpr (SYNC) {
                if (i == NS - 2 * NQ) handover();
            }
            sn.s[kb][qb] = mfma16(ka[op % NQ], qB[qb][ks], ks == 0 ? negm[qb] : sn.s[kb][qb]);
            if (i & 1) {
                if (op + NQ < NOP) load_k(K1, op + NQ, op % NQ);
                else load_v(op + NQ - NOP, op % NQ);
            }
            if constexpr (NS == 16) { if ((i & 1) == 0) exp_pair(i >> 1); }
            else exp_pair(i);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- phase B ----
        bool due = false;
        int mx = 0;
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int db = i >> 1, qb = (i & 1) ^ (db & 1);
            oacc[db][qb] = mfma16(va[db % NQ], pB[qb], oacc[db][qb]);
            if (i & 1) {
                if (db + NQ < NOP) load_v(db + NQ, db % NQ);
                else load_k(K2, db + NQ - NOP, db % NQ);
            }
            constexpr int R0 = NS / 2 - (NS >= 16 ? 3 : 2);
            if (i == R0) { if (MAYMASK && masked_next) mask_block(sn, key0_next); }
            if (i >= R0 && i < R0 + 4) mx = max_piece(sn, i - R0, mx);
            if (i == R0 + 3) due = __builtin_amdgcn_ballot_w64(mx > 0x41000000) != 0;       // 8.0f
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) lacc[qb] = mfma16(ones8, pB[qb], lacc[qb]);
        if (due) rescale(sn);
    };

    // ---- prologue: K stages 0 and 1 and V stage 0; scores of block 0; first K operands of block 1 ----
    TRN_FETCH_K(0, Ks0);
    TRN_FETCH_V(0, Vs0);
    if (ntiles > 1) TRN_FETCH_K(1, Ks1);

    // ---- Q^T B-operands: lane holds Q[qrow[qb]][32 ks + 8 g4 .. +7].  The loads go out behind the first K/V stage
    // fetches and all together, so that the workgroup's start-up pays one memory latency, not three in a row.
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const int qrow_ld = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;       // clamp loads; stores are predicated
        const half_t* qp = a.q + b * a.qb + head * a.qh + (int64_t)qrow_ld * a.qs + 8 * g4;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) qB[qb][ks] = *reinterpret_cast<const half8_t*>(qp + ks * 32);
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const bool q_norm = a.q_norm != 0;
        if (q_norm) {   // fused per-head RMSNorm of the query row (the rest of the row is in the lanes n + 16, + 32, + 48)
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e) { float f = (float)qB[qb][ks][e]; ss += f * f; }
            ss = quad_sum(ss);
            const float rstd = 1.0f / __builtin_sqrtf(ss / (float)D + a.q_eps);
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                half8_t gq;
                if (a.gamma_q) gq = *reinterpret_cast<const half8_t*>(a.gamma_q + ks * 32 + 8 * g4);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float y = (float)qB[qb][ks][e] * rstd;
                    if (a.gamma_q) y = (float)gq[e] * y;
                    qB[qb][ks][e] = (half_t)y;
                }
            }
        }
        // the softmax scale and log2(e) go into Q once, so that the scores leave the matrix pipe ready for exp2
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) qB[qb][ks][e] = (half_t)((float)qB[qb][ks][e] * a.c1);
    }

    __builtin_amdgcn_s_waitcnt(0x0f70);     // vmcnt(0): this wave's loads have landed in LDS
    __syncthreads();

    Scores16 sA, sB;                        // scores of the current / next 32-key block (ping-pong)
    {
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const half8_t k0 = *reinterpret_cast<const half8_t*>(&Ks0[kb * 16 * D + koff[ks]]);
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) sA.s[kb][qb] = mfma16(k0, qB[qb][ks], ks == 0 ? zero : sA.s[kb][qb]);
            }
#pragma unroll
        for (int i = 0; i < NQ; ++i) load_k(Ks0 + 32 * D, i, i);
        // block 0 sets the reference outright (every query sees key 0, so it is finite from here on)
        float smax[2];
        mask_block(sA, 0);
        block_max(sA, smax);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            m[qb] = quad_max(smax[qb]);
            negm[qb] = float4_t{-m[qb], -m[qb], -m[qb], -m[qb]};
            sA.s[0][qb] = sA.s[0][qb] - m[qb];
            sA.s[1][qb] = sA.s[1][qb] - m[qb];
        }
    }

    // One 64-key tile jt.  Kc = its own K stage (block 1 still has operands to give), Kn = the next tile's
    // K stage, Vc = its V stage, Vn = the other V stage.
    auto tile = [&](auto maymask_tag, int jt, half_t* Kc, const half_t* Kn, const half_t* Vc, half_t* Vn) __attribute__((always_inline)) {
        const int kv0 = jt * BN;
        auto handover = [&]() __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt(0x0f70);   // this wave's share of stages Kn and Vc is in LDS
            __syncthreads();                      // ... and everyone's; Kc and Vn have had their last readers
            // (unconditional: tiles past the end of the keys read as zeros into stages nobody reads, and the
            // hand-over stays free of branches)
            TRN_FETCH_K(jt + 2, Kc);
            TRN_FETCH_V(jt + 1, Vn);
        };
        auto none = [&]() __attribute__((always_inline)) {};
        // (Past the last tile a K stage holds stale rows; scores computed from them are masked away.)
        step(needs_mask(kv0 + 32), maymask_tag, std::true_type{}, sA, sB, Vc, Kc + 32 * D, Kn, kv0 + 32, handover);
        step(needs_mask(kv0 + 64), maymask_tag, std::false_type{}, sB, sA, Vc + 32 * D, Kn, Kn + 32 * D, kv0 + 64, none);
    };
    // Under a causal mask the waves of a workgroup see different numbers of tiles: a wave computes the tiles that
    // hold a key visible to one of its queries, and for the rest only keeps up the staging it shares with the
    // others (its part of every refill, and the barrier), leaving its SIMD to the wave that still computes.
    int nlive = ntiles;
    if (a.causal) nlive = min(ntiles, (min(wq0 + 31, a.Sq - 1) + off) / BN + 1);
    if (idle) nlive = 0;
    // The leading tiles whose blocks (and the first block of the tile after) lie wholly inside the keys and, under a
    // causal mask, before this wave's first query: a loop of their own without the mask test.  needs_mask is monotone
    // in the key index, so they are the tiles jt with 64 jt + 96 <= Skv and 64 jt + 95 <= wb; taken in pairs (the
    // stages alternate), the rest goes through the general loop.
    int n_plain = (a.Skv - 96 >= 0) ? (a.Skv - 96) / BN + 1 : 0;
    if (a.causal) n_plain = min(n_plain, wb - 95 >= 0 ? (wb - 95) / BN + 1 : 0);
    n_plain = min(n_plain, nlive) & ~1;
    for (int jt = 0; jt < n_plain; jt += 2) {
        tile(std::false_type{}, jt, Ks0, Ks1, Vs0, Vs1);
        tile(std::false_type{}, jt + 1, Ks1, Ks0, Vs1, Vs0);
    }
    for (int jt = n_plain; jt < nlive; jt += 2) {
        tile(std::true_type{}, jt, Ks0, Ks1, Vs0, Vs1);
        if (jt + 1 < nlive) tile(std::true_type{}, jt + 1, Ks1, Ks0, Vs1, Vs0);
    }
    for (int jt = nlive; jt < ntiles; ++jt) {
        half_t* Kc = (jt & 1) ? Ks1 : Ks0;
        half_t* Vn = (jt & 1) ? Vs0 : Vs1;
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (jt + 2 < ntiles) TRN_FETCH_K(jt + 2, Kc);
        if (jt + 1 < ntiles) TRN_FETCH_V(jt + 1, Vn);
    }
#undef TRN_FETCH_K
#undef TRN_FETCH_V

    // ---- epilogue: normalise; transpose this wave's 32 x D tile through LDS so that the stores are whole
    // 16-byte-per-lane row segments; LSEs ----
    float inv[2];
    float l[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { l[qb] = lacc[qb][0]; inv[qb] = 1.0f / l[qb]; }
    __builtin_amdgcn_s_waitcnt(0x0f70);                // this wave's last refills (past the end, unread) have landed ...
    __syncthreads();                                   // ... and everyone's; every wave is done with the K/V stages
    {
        // two passes of D/2 columns each, so that NW waves' staging regions fit in the four stage arrays
        constexpr int DP = D / 2, OP = DP + 4;         // row pitch in halfs
        constexpr int LPRW = DP / 8, RPS = 64 / LPRW;  // lanes per output row segment, rows per store instruction
        static_assert(32 * OP * 2 <= BN * D * 2 / (NW / 4), "staging region too large");
        half_t* arr = (wave / (NW / 4)) == 0 ? Ks0 : (wave / (NW / 4)) == 1 ? Ks1 : (wave / (NW / 4)) == 2 ? Vs0 : Vs1;
        half_t* ot = arr + (wave % (NW / 4)) * (BN * D / (NW / 4));
        const int orow = lane / LPRW, ocol = (lane % LPRW) * 8;
        half_t* ob = a.o + b * a.ob + head * a.oh;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
            for (int dbl = 0; dbl < NOP / 2; ++dbl)
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    half4_t ov;
#pragma unroll
                    for (int e = 0; e < 4; ++e) ov[e] = (half_t)(oacc[pass * (NOP / 2) + dbl][qb][e] * inv[qb]);
                    *reinterpret_cast<half4_t*>(&ot[(16 * qb + n) * OP + dbl * 16 + 4 * g4]) = ov;
                }
            // (LDS operations of one wave execute in order: no wait needed between its own writes and reads)
#pragma unroll
            for (int jj = 0; jj < 32 / RPS; ++jj) {
                const int r = jj * RPS + orow;
                const uint2_t lo = *reinterpret_cast<const uint2_t*>(&ot[r * OP + ocol]);
                const uint2_t hi = *reinterpret_cast<const uint2_t*>(&ot[r * OP + ocol + 4]);
                if (wq0 + r < a.Sq)
                    *reinterpret_cast<uint4_t*>(ob + (int64_t)(wq0 + r) * a.os + pass * DP + ocol) = uint4_t{lo.x, lo.y, hi.x, hi.y};
            }
        }
    }
    if (g4 == 0 && a.lse) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
            if (qrow[qb] < a.Sq) a.lse[((int64_t)b * a.Hq + head) * a.Sq + qrow[qb]] = (m[qb] + fast_log2(l[qb])) * kLn2;
    }
#endif
}

template <int D, int NW, bool PAIRED = false>
static hipError_t launch16(AttnArgs a, hipStream_t s) {
    int64_t grid;
    if (PAIRED) {
        a.n_qtiles = (a.Sq + 127) / 128;
        grid = (int64_t)((a.n_qtiles + 1) / 2) * a.B * a.Hq;
    } else {
        a.n_qtiles = (a.Sq + 32 * NW - 1) / (32 * NW);
        grid = (int64_t)a.n_qtiles * a.B * a.Hq;
    }
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((attn_fwd16_kernel<D, NW, PAIRED>), dim3((unsigned)grid), dim3(NW * 64), 0, s, a);
    return hipGetLastError();
}

// Workgroup shape by problem size.  Wide (each K/V stage is fetched from L2 once per 256 queries: a few % less energy,
// and this kernel is power-limited) when that still fills the chip: one workgroup per CU for unmasked attention; under
// a causal mask workgroups differ in length by up to n_qtiles x, so at least two rounds are needed to balance (measured
// at 512 wide workgroups: +2.3 % with head_dim 128; with head_dim 64 the wide form loses 10-20 % at every size).  A
// causal problem whose narrow workgroups would all be resident at once (a single round: the longest tile sets the time,
// twice the mean) runs paired instead, which gives every workgroup the same work -- if the pairs still cover the chip.
Attn16Shape attn_fwd16_shape(int batch, int n_q_heads, int seq_q, int head_dim, bool causal) {
    const int64_t bh = (int64_t)batch * n_q_heads;
    const int64_t n128 = (seq_q + 127) / 128;
    // (paired workgroups are half as many: below about three quarters of the CUs the idle ones cost more than the
    // imbalance -- measured at 1024 queries x 32 heads: 22.9 us narrow, 24.8 us paired; at 2048: 46.3 and 43.1)
    if (causal && n128 * bh <= 512 && ((n128 + 1) / 2) * bh >= 192) return Attn16Shape::Paired;
    const int64_t n_wide = (int64_t)((seq_q + 255) / 256) * bh;
    return head_dim == 128 && n_wide >= (causal ? 512 : 256) ? Attn16Shape::Wide : Attn16Shape::Narrow;
}

hipError_t launch_attn_fwd16(const AttnArgs& a, int head_dim, Attn16Shape shape, hipStream_t s) {
    if (shape == Attn16Shape::Paired) return head_dim == 128 ? launch16<128, 8, true>(a, s) : launch16<64, 8, true>(a, s);
    const bool wide = shape == Attn16Shape::Wide;
    if (head_dim == 128) return wide ? launch16<128, 8>(a, s) : launch16<128, 4>(a, s);
    return wide ? launch16<64, 8>(a, s) : launch16<64, 4>(a, s);
}

const char* attn_fwd16_kernel_name(int head_dim, Attn16Shape shape) {
    if (shape == Attn16Shape::Paired) return head_dim == 128 ? "trn::attn_fwd16_kernel<128, 8, true>" : "trn::attn_fwd16_kernel<64, 8, true>";
    const bool wide = shape == Attn16Shape::Wide;
    if (head_dim == 128) return wide ? "trn::attn_fwd16_kernel<128, 8, false>" : "trn::attn_fwd16_kernel<128, 4, false>";
    return wide ? "trn::attn_fwd16_kernel<64, 8, false>" : "trn::attn_fwd16_kernel<64, 4, false>";
}

}  // namespace trn
