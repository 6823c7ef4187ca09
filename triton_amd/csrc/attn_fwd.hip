// Flash attention forward for gfx950 on the 32x32x16 MFMA: O = softmax(scale * Q K^T [+causal]) V, GQA/MQA,
// head_dim 64/128.  This file holds the entry points, and the kernel that runs when the scores are perturbed
// (KeyFormer: one lane owns a whole query row here, which is what the noise stream wants); plain attention runs
// on the 16x16x32 kernel of attn_fwd16.hip.
//
// Formulation.  Everything is computed TRANSPOSED so that a lane owns one query:
//     S^T[key][query] = K[key][:] . Q[query][:]     (MFMA 32x32x16: A = K tile from LDS, B = Q^T in registers)
//     O^T[d][query]  += V^T[d][key] * P^T[key][query]   (A = V^T tile from LDS, B = P^T straight from the
//                                                         S^T accumulator registers, rounded to fp16)
// In the 32x32 accumulator layout lane l holds column l%32 (the query) and 16 of the 32 rows (keys), so the
// softmax row max / row sum are in-lane reductions plus ONE exchange with lane l^32, the running max and
// normaliser are one scalar per lane, the O rescale needs no shuffles, and P never touches LDS: the MFMA
// contraction index may be permuted freely, so the accumulator's key order is matched by the order in
// which V^T is fetched.
//
// Workgroup: 256 threads = 4 waves, 128 queries (32 per wave); K/V tiles of BN keys go straight from global
// memory into double-buffered LDS (buffer_load ... lds, no register staging), row-major with an XOR chunk
// swizzle; the V^T A-operand is fetched with the gfx950 transposing LDS read ds_read_b64_tr_b16, so V needs
// no transposition in memory or on the way in.
// Grid: one workgroup per (query tile, batch, head), heaviest (latest) query tiles first; consecutive
// workgroup ids map to different KV heads so that the query heads sharing a KV head land on the same XCD
// (ids are dealt round-robin to the 8 XCDs) and hit its L2.
#include "attn.h"
#include <type_traits>

namespace trn {

template <int D, int NW, bool NOISE>
__global__ __launch_bounds__(NW * 64, NW == 8 ? 1 : 2) void attn_fwd_kernel(const AttnArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-descriptor types and LDS-load builtins exist in the device pass only;
                                      // the host pass needs just the launch stub
    constexpr int BN = 64;       // keys per LDS stage (two 32-key blocks)
    constexpr int NS = D / 16;   // MFMA slots per phase: k-steps of S^T = K Q^T, and (2 key halves) x (D/32) of P V
    constexpr int NDB = D / 32;  // 32-wide blocks of head_dim in O^T
    constexpr int EPI = 16 / NS; // score elements converted per slot
    constexpr int CPR = D / 8;   // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;            // stage rows covered by one wave-wide 1 KB load
    constexpr int NI = BN / (RPI * NW);      // such loads per wave per stage (K and V each)
    constexpr int BM = 32 * NW;              // queries per workgroup: NW waves x 32
    // Two stages each for K and V, as FOUR separate arrays: the compiler orders an LDS read after every
    // outstanding global->LDS load that may alias it, and only distinct variables are provably disjoint --
    // with one [2][..] array every LDS read would wait for the prefetch that was just issued.
    __shared__ __attribute__((aligned(1024))) half_t Ks0[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Ks1[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Vs0[BN * D];
    __shared__ __attribute__((aligned(1024))) half_t Vs1[BN * D];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- which (query tile, batch, head): heavy tiles first, KV heads interleaved across ids
    const int BH = a.B * a.Hq;
    const int qt = a.n_qtiles - 1 - (int)(blockIdx.x / BH);
    const int j = blockIdx.x % BH;
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;

    const int off = a.Skv - a.Sq;                       // causal: query i sees keys <= i + off
    const int q0 = qt * BM;
    const int wq0 = q0 + wave * 32;                     // first query of this wave
    const int qrow = wq0 + c;                           // this lane's query
    const int qrow_ld = qrow < a.Sq ? qrow : a.Sq - 1;  // clamp loads; stores are predicated

    // ---- Q^T B-operands: lane holds Q[qrow][ks*16 + 8h .. +7]
    half8_t qB[NS];
    {
        const half_t* qp = a.q + b * a.qb + head * a.qh + (int64_t)qrow_ld * a.qs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < NS; ++ks) qB[ks] = *reinterpret_cast<const half8_t*>(qp + ks * 16);
        if (a.q_norm) {   // fused per-head RMSNorm of the query row (other half of the row is in lane^32)
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < NS; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e) { float f = (float)qB[ks][e]; ss += f * f; }
            ss = half_sum(ss);
            const float rstd = 1.0f / __builtin_sqrtf(ss / (float)D + a.q_eps);
#pragma unroll
            for (int ks = 0; ks < NS; ++ks) {
                half8_t gq;
                if (a.gamma_q) gq = *reinterpret_cast<const half8_t*>(a.gamma_q + ks * 16 + 8 * h);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float y = (float)qB[ks][e] * rstd;
                    if (a.gamma_q) y = (float)gq[e] * y;
                    qB[ks][e] = (half_t)y;
                }
            }
        }
    }

    // ---- LDS read offsets (halfs), lane constants.  K operand: row c of a 32-key block, logical chunk 2ks+h.
    int koff[NS];
#pragma unroll
    for (int ks = 0; ks < NS; ++ks) koff[ks] = c * D + (((2 * ks + h) ^ swz<D>(c)) << 3);
    // V^T operand through the transposing read: in each 16-lane group lanes 4r..4r+3 supply stage row r
    // (4 consecutive 8-byte pieces); this lane's piece is row 4h + (lane%16)/4 [+8], head_dim columns
    // db*32 + 16*((lane/16)%2) + 4*(lane%4).
    int voff_lo[NDB], voff_hi[NDB];
    {
        const int rl = 4 * h + ((lane & 15) >> 2), rh = rl + 8;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            voff_lo[db] = rl * D + (((db * 4 + lc) ^ swz<D>(rl)) << 3) + sub;
            voff_hi[db] = rh * D + (((db * 4 + lc) ^ swz<D>(rh)) << 3) + sub;
        }
    }

    float16_t oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;      // reference max (log2 domain) and this lane's partial row sum
    float m2 = 0.f, l2 = 0.f;          // same for the perturbed scores: reference (finite; meaningful once have2) and sum
    bool have2 = false;

    int ntiles = (a.Skv + BN - 1) / BN;
    if (a.causal) ntiles = min(ntiles, (min(q0 + BM - 1, a.Sq - 1) + off) / BN + 1);

    // KeyFormer noise: this lane's query row, the 4 x 4 keys of its accumulator layout per 32-key block.  It is
    // the HBM stream that bounds that variant, so each block's 64 bytes per lane are requested two pipeline steps
    // before they are used (buffer loads: keys or rows past the end read as zeros and are masked anyway).
    const __amdgpu_buffer_rsrc_t nrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(NOISE ? a.noise + b * a.nb + head * a.nh : nullptr), 0,
        NOISE ? (int)(((int64_t)(a.Sq - 1) * a.ns + a.Skv) * 4) : 0, 0x00020000);
    const int nvo = NOISE ? (int)(((int64_t)qrow_ld * a.ns + 4 * h) * 4) : 0;
    float4_t gpre0[4], gpre1[4];       // even / odd 32-key blocks: each refilled two blocks ahead, as soon as it is used
    auto fetch_noise = [&](int key0, float4_t (&gpre)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
            gpre[r4] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(nrs, nvo + r4 * 32, key0 * 4, 0));
    };

    // ---- staging: direct global -> LDS loads.  Buffer descriptors give zero fill for keys past the end
    // (an all-zero V row times P = 0 contributes nothing; garbage could be NaN).
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.k + b * a.kb + kvh * a.kh), 0, (int)(((int64_t)(a.Skv - 1) * a.ks + D) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.v + b * a.vb + kvh * a.vh), 0, (int)(((int64_t)(a.Skv - 1) * a.vs + D) * 2), 0x00020000);
    const int st_row = wave * RPI + lane / CPR;                      // this lane's row within each 4*RPI-row group
    const int st_chunk = (lane % CPR) ^ swz<D>(st_row);             // LDS slot lane%CPR of that row holds this logical chunk
    const int kvo = (int)(st_row * a.ks * 2) + st_chunk * 16;       // per-lane byte offsets within a stage
    const int vvo = (int)(st_row * a.vs * 2) + st_chunk * 16;
    const int krow_bytes = (int)(RPI * a.ks * 2), vrow_bytes = (int)(RPI * a.vs * 2);
    const int ktile_bytes = (int)(BN * a.ks * 2), vtile_bytes = (int)(BN * a.vs * 2);
#define TRN_FETCH_K(jt_, dst_) fetch_tile<NI, D, NW>(krs, &dst_[wave * RPI * D], kvo, (jt_) * ktile_bytes, krow_bytes)
#define TRN_FETCH_V(jt_, dst_) fetch_tile<NI, D, NW>(vrs, &dst_[wave * RPI * D], vvo, (jt_) * vtile_bytes, vrow_bytes)

    const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int wb = wq0 + off;          // key index bound of this wave's first query
    auto needs_mask = [&](int key0) { return (key0 + 32 > a.Skv) || (a.causal && key0 + 31 > wb); };

    // Scores of a 32-key block starting at key0, just produced: (KeyFormer) fold them into the perturbed
    // row normaliser; mask; block max against the LAZY reference max m.  m is only raised when some row's
    // true running max exceeds it by more than 2^8: probabilities are then at most 256 (exact in fp16's
    // range, fp32 sums), O and l stay relative to the same m so the final O/l and m + log2(l) are unchanged,
    // and the 16*NDB-multiply rescale of O^T runs on the first block or two only instead of on most blocks.
    // Returns whether a rescale is due (wave-uniform) and the candidate max.
    auto reduce_block = [&](bool masked, float16_t& sx, int key0, float& smax, float4_t (&gpre)[4]) __attribute__((always_inline)) {
        // `masked` is wave-uniform: the branches below touch only this block's 16 score registers, so the
        // accumulators never meet a control-flow merge.  (Two whole-step variants selected by a branch cost
        // dozens of accumulator register copies per step and broke the in-place MFMA accumulation chains.)
        if constexpr (NOISE) {
            // Row normaliser of the perturbed scores z = s*c2 + g*c3 (log2 domain), with a lazy reference like the
            // main softmax: d = z - m2 comes straight out of two fused multiply-adds, and m2 is only raised when some d
            // exceeds 8 (the sum lives in fp32: 2^8 of head-room is harmless) or nothing has been summed yet.
            const float nref = -m2;
            float16_t d;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const float4_t gv = gpre[r4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float dd = __builtin_fmaf(sx[r4 * 4 + e], a.c2, __builtin_fmaf(gv[e], a.c3, nref));
                    if (masked) {
                        const int key = key0 + 8 * r4 + 4 * h + e;
                        dd = (key < a.Skv && (!a.causal || key <= qrow + off)) ? dd : -INFINITY;
                    }
                    d[r4 * 4 + e] = dd;
                }
            }
            fetch_noise(key0 + 64, gpre);    // the next block of the same parity, two pipeline steps ahead of its use
            // The test runs on the lane's own 16 keys; the exchange with the other lane of the query (m2 and have2 are
            // shared by the pair) is made on the rare path only -- if either lane of a pair wants the raise, the
            // wave-wide vote takes every lane there.
            const float down = max16_bare(d);
            if (__builtin_amdgcn_ballot_w64(down > 8.0f || (!have2 && down > -INFINITY)) != 0) {     // rare after a row's first block
                const float dmax = half_max(down);
                const bool seen = dmax > -INFINITY;            // a block can be entirely masked for this row pair
                const bool raise = dmax > 8.0f || (!have2 && seen);
                const float shift = raise ? dmax : 0.f;
                l2 *= fast_exp2(-shift);
                m2 += shift;
#pragma unroll
                for (int r = 0; r < 16; ++r) d[r] -= shift;
                have2 = have2 || seen;
            }
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += fast_exp2(d[r]);
            l2 += sum;
        }
        if (masked) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r / 4) + 4 * h + (r % 4);
                const bool ok = key < a.Skv && (!a.causal || key <= qrow + off);
                sx[r] = ok ? sx[r] : -INFINITY;      // (a select: stale-LDS garbage past the last block never propagates)
            }
        }
        smax = max16_bare(sx) * a.c1;          // over the lane's own keys; the pair's maximum is formed in rescale()
        return __builtin_amdgcn_ballot_w64(smax > m + 8.0f) != 0;
    };
    auto rescale = [&](float smax_own) __attribute__((always_inline)) {
        const float smax = half_max(smax_own);
        const float mnew = fmaxf(m, smax);
        const float alpha = fast_exp2(m - mnew);
        l *= alpha;
#pragma unroll
        for (int i = 0; i < NDB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
        m = mnew;
    };

    constexpr int NQ = 2;   // operand look-ahead in MFMA slots (deeper windows measured the same)
    half8_t ka[NQ];    // K operands of the next block's S^T: a rolling window NQ MFMA slots ahead of use
    half8_t va[NQ];    // V^T operands of this block's P V: likewise

    // One pipeline step for block B whose scores sc are complete, masked and reflected in m:
    //   phase A: MFMA: S^T of block B+1                  | VALU: P = exp2(sc*c1 - m), fp16, row sum
    //   phase B: MFMA: O^T += V^T P^T                    | VALU: mask + max of block B+1's scores
    // A wave issues in order and an MFMA holds the matrix pipe for 8 passes, so program order IS the
    // schedule: one MFMA, its share of the VALU work and one LDS operand request per slot, with
    // sched_barrier to keep the compiler from regrouping.  Each operand is requested NQ slots before its
    // MFMA, into the register its predecessor just vacated:
    //   phase A slot i < NS-NQ : K operand i+NQ of block B+1 (K1)   later slots : V^T operand i+NQ-NS of block B
    //   phase B slot i < NS-NQ : V^T operand i+NQ of block B        later slots : K operand i+NQ-NS of block B+2 (K2)
    // With SYNC (first block of a 64-key tile) the tile hand-over sits NQ slots before the end of phase A: by
    // then every wave has made its last read of the tile's own K stage (block B+1's last operands) and of the
    // previous tile's V stage, so after the barrier those two stages are refilled (K two tiles ahead, V one
    // tile ahead) and all later LDS reads of this and the next step go to the stages that just became visible.
    auto step = [&](bool masked_next, auto sync_tag, float16_t& sc, float16_t& sn, const half_t* Vblk, const half_t* K1,
                    const half_t* K2, int key0_next, auto&& handover) __attribute__((always_inline)) {
        constexpr bool SYNC = decltype(sync_tag)::value;
        // The row sum is taken over the fp16-rounded P (v_dot2_f32_f16 against ones, fp32 accumulate),
        // i.e. over exactly the values that multiply V.
        const half2_t ones = {(half_t)1.f, (half_t)1.f};
        half8_t pB[2];
        auto load_v = [&](int op, int reg) __attribute__((always_inline)) {
            const half_t* vp = Vblk + 16 * (op / NDB) * D;
            half4_t lo = lds_read_tr16(vp + voff_lo[op % NDB]);   // keys +0..3 of this lane half, dim db*32+c
            half4_t hi = lds_read_tr16(vp + voff_hi[op % NDB]);   // keys +8..11
            va[reg] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        // ---- phase A ----
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            if constexpr (SYNC) {
                if (i == NS - NQ) handover();
            }
            sn = mfma32(ka[i % NQ], qB[i], i == 0 ? zero : sn);
            if (i + NQ < NS) ka[i % NQ] = *reinterpret_cast<const half8_t*>(&K1[koff[i + NQ]]);
            else load_v(i + NQ - NS, i % NQ);
#pragma unroll
            for (int e = 0; e < EPI; e += 2) {
                const int r = i * EPI + e;
                const float p0 = fast_exp2(__builtin_fmaf(sc[r], a.c1, -m));
                const float p1 = fast_exp2(__builtin_fmaf(sc[r + 1], a.c1, -m));
                const half2_t pp = {(half_t)p0, (half_t)p1};
                l = __builtin_amdgcn_fdot2(pp, ones, l, false);
                pB[r / 8][r % 8] = pp[0]; pB[r / 8][r % 8 + 1] = pp[1];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- phase B ----
        float smax = 0.f;
        bool due = false;
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            oacc[i % NDB] = mfma32(va[i % NQ], pB[i / NDB], oacc[i % NDB]);
            if (i + NQ < NS) load_v(i + NQ, i % NQ);
            else ka[i % NQ] = *reinterpret_cast<const half8_t*>(&K2[koff[i + NQ - NS]]);
            if (i == NS / 2) due = reduce_block(masked_next, sn, key0_next, smax, SYNC ? gpre1 : gpre0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (due) rescale(smax);
    };

    // ---- prologue: K stages 0 and 1 and V stage 0; scores of block 0; first K operands of block 1 ----
    if constexpr (NOISE) { fetch_noise(0, gpre0); fetch_noise(32, gpre1); }
    TRN_FETCH_K(0, Ks0);
    TRN_FETCH_V(0, Vs0);
    if (ntiles > 1) TRN_FETCH_K(1, Ks1);
    __builtin_amdgcn_s_waitcnt(0x0f70);     // vmcnt(0): this wave's loads have landed in LDS
    __syncthreads();

    float16_t sA, sB;                       // scores of the current / next 32-key block (ping-pong)
    {
        half8_t k0[NS];
#pragma unroll
        for (int i = 0; i < NS; ++i) k0[i] = *reinterpret_cast<const half8_t*>(&Ks0[koff[i]]);
#pragma unroll
        for (int i = 0; i < NS; ++i) sA = mfma32(k0[i], qB[i], i == 0 ? zero : sA);
#pragma unroll
        for (int i = 0; i < NQ; ++i) ka[i] = *reinterpret_cast<const half8_t*>(&Ks0[32 * D + koff[i]]);
        float smax;
        if (reduce_block(true, sA, 0, smax, gpre0)) rescale(smax);
    }

    // One 64-key tile jt.  Kc = its own K stage (block 1 still has operands to give), Kn = the next tile's
    // K stage, Vc = its V stage, Vn = the other V stage.
    auto tile = [&](int jt, half_t* Kc, const half_t* Kn, const half_t* Vc, half_t* Vn) __attribute__((always_inline)) {
        const int kv0 = jt * BN;
        auto handover = [&]() __attribute__((always_inline)) {
            // this wave's share of stages Kn and Vc is in LDS: everything but the noise requests of the two
            // steps since the stages were requested (2 x 4 loads, issued behind them) has returned
            if constexpr (NOISE) __builtin_amdgcn_s_waitcnt(0x0f78); else __builtin_amdgcn_s_waitcnt(0x0f70);
            __syncthreads();                      // ... and everyone's; Kc and Vn have had their last readers
            // With noise in flight the refills are issued unconditionally (tiles past the end just fill stages
            // nobody reads): the compiler sizes its waits for the noise registers by the loads it KNOWS follow
            // them, and a conditional load counts as absent -- every noise use would drain the refills too.
            if (NOISE || jt + 2 < ntiles) TRN_FETCH_K(jt + 2, Kc);
            if (NOISE || jt + 1 < ntiles) TRN_FETCH_V(jt + 1, Vn);
        };
        auto none = [&]() __attribute__((always_inline)) {};
        // (Past the last tile a K stage holds stale rows; scores computed from them are masked away.)
        step(needs_mask(kv0 + 32), std::true_type{}, sA, sB, Vc, Kc + 32 * D, Kn, kv0 + 32, handover);
        step(needs_mask(kv0 + 64), std::false_type{}, sB, sA, Vc + 32 * D, Kn, Kn + 32 * D, kv0 + 64, none);
    };
    for (int jt = 0; jt < ntiles; jt += 2) {
        tile(jt, Ks0, Ks1, Vs0, Vs1);
        if (jt + 1 < ntiles) tile(jt + 1, Ks1, Ks0, Vs1, Vs0);
    }
#undef TRN_FETCH_K
#undef TRN_FETCH_V

    // ---- epilogue: normalise; transpose this wave's 32 x D tile through LDS so that the stores are whole
    // 16-byte-per-lane row segments (the accumulator layout would give 8-byte pieces scattered over 32 rows,
    // i.e. partial-line writes); LSEs ----
    l = half_sum(l);
    const float inv = 1.0f / l;
    __syncthreads();                                   // every wave is done with the K/V stages
    {
        // two passes of D/2 columns each, so that NW waves' staging regions fit in the four stage arrays
        constexpr int DP = D / 2, OP = DP + 4;         // row pitch in halfs: 8-byte writes of 32 rows spread over all banks
        constexpr int LPRW = DP / 8, RPS = 64 / LPRW;  // lanes per output row segment, rows per store instruction
        static_assert(32 * OP * 2 <= BN * D * 2 / (NW / 4), "staging region too large");
        half_t* arr = (wave / (NW / 4)) == 0 ? Ks0 : (wave / (NW / 4)) == 1 ? Ks1 : (wave / (NW / 4)) == 2 ? Vs0 : Vs1;
        half_t* ot = arr + (wave % (NW / 4)) * (BN * D / (NW / 4));
        const int orow = lane / LPRW, ocol = (lane % LPRW) * 8;
        half_t* ob = a.o + b * a.ob + head * a.oh;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
            for (int dbl = 0; dbl < NDB / 2; ++dbl)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    half4_t ov;
#pragma unroll
                    for (int e = 0; e < 4; ++e) ov[e] = (half_t)(oacc[pass * (NDB / 2) + dbl][r4 * 4 + e] * inv);
                    *reinterpret_cast<half4_t*>(&ot[c * OP + dbl * 32 + 8 * r4 + 4 * h]) = ov;
                }
            // (LDS operations of one wave execute in order: no wait needed between its own writes and reads)
#pragma unroll
            for (int j = 0; j < 32 / RPS; ++j) {
                const int r = j * RPS + orow;
                const uint2_t lo = *reinterpret_cast<const uint2_t*>(&ot[r * OP + ocol]);
                const uint2_t hi = *reinterpret_cast<const uint2_t*>(&ot[r * OP + ocol + 4]);
                if (wq0 + r < a.Sq)
                    *reinterpret_cast<uint4_t*>(ob + (int64_t)(wq0 + r) * a.os + pass * DP + ocol) = uint4_t{lo.x, lo.y, hi.x, hi.y};
            }
        }
    }
    if (qrow < a.Sq && h == 0 && a.lse) a.lse[((int64_t)b * a.Hq + head) * a.Sq + qrow] = (m + fast_log2(l)) * kLn2;
    if constexpr (NOISE) {
        const float l2s = half_sum(l2);
        if (qrow < a.Sq && h == 0)
            a.lse_pert[((int64_t)b * a.Hq + head) * a.Sq + qrow] = (m2 + fast_log2(l2s)) * kLn2;
    }
#endif
}

template <int D, int NW, bool NOISE>
static hipError_t launch_fwd(AttnArgs a, hipStream_t s) {
    a.n_qtiles = (a.Sq + 32 * NW - 1) / (32 * NW);
    const int64_t grid = (int64_t)a.n_qtiles * a.B * a.Hq;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((attn_fwd_kernel<D, NW, NOISE>), dim3((unsigned)grid), dim3(NW * 64), 0, s, a);
    return hipGetLastError();
}

int validate_attn(const trn_attn_desc* d, bool need_v);
int validate_attn(const trn_attn_desc* d, bool need_v) {
    if (d->batch <= 0 || d->n_q_heads <= 0 || d->n_kv_heads <= 0 || d->seq_q <= 0 || d->seq_kv <= 0) return TRN_E_SHAPE;
    if (d->n_q_heads % d->n_kv_heads != 0) return TRN_E_SHAPE;
    if (d->head_dim != 64 && d->head_dim != 128) return TRN_E_UNSUPPORTED;
    if (d->causal && d->seq_kv < d->seq_q) return TRN_E_SHAPE;
    if (!(d->scale > 0.f)) return TRN_E_UNSUPPORTED;
    const int64_t D = d->head_dim;
    if (d->q_stride_s < D || d->k_stride_s < D) return TRN_E_STRIDE;
    if (need_v && (d->v_stride_s < D || d->o_stride_s < D)) return TRN_E_STRIDE;
    const int64_t st[] = {d->q_stride_b, d->q_stride_h, d->q_stride_s, d->k_stride_b, d->k_stride_h, d->k_stride_s};
    for (int64_t x : st) if (x < 0 || !pitch16(x, 2)) return TRN_E_ALIGN;
    if (need_v) {
        const int64_t sv[] = {d->v_stride_b, d->v_stride_h, d->v_stride_s, d->o_stride_b, d->o_stride_h, d->o_stride_s};
        for (int64_t x : sv) if (x < 0 || !pitch16(x, 2)) return TRN_E_ALIGN;
    }
    return TRN_OK;
}

}  // namespace trn

namespace trn {
// Workgroup shape of the forward kernel with score perturbation: 8 waves x 32 queries when that still fills the chip.
static bool noise_kernel_wide(const trn_attn_desc* d) {
    const int64_t n_wide = (int64_t)((d->seq_q + 255) / 256) * d->batch * d->n_q_heads;
    return n_wide >= (!d->causal ? 256 : d->head_dim == 128 ? 512 : 1024);
}
}  // namespace trn

extern "C" int64_t trn_attn_workspace_bytes(const trn_attn_desc* d) {
    using namespace trn;
    if (!d || validate_attn(d, true) != TRN_OK) return 0;
    return attn_decode_workspace_bytes(d->batch, d->n_q_heads, d->seq_q, d->seq_kv, d->head_dim);
}

extern "C" const char* trn_attn_fwd_kernel_name(const trn_attn_desc* d, int32_t with_noise) {
    using namespace trn;
    if (!d || validate_attn(d, true) != TRN_OK) return "";
    const bool d128 = d->head_dim == 128;
    if (d->seq_q <= 32) return attn_decode_kernel_name(d->batch, d->n_q_heads, d->seq_kv, d->head_dim, with_noise != 0);
    if (!with_noise) return attn_fwd16_kernel_name(d->head_dim, attn_fwd16_shape(d->batch, d->n_q_heads, d->seq_q, d->head_dim, d->causal != 0));
    const bool wide = noise_kernel_wide(d);
    if (d128) return wide ? "trn::attn_fwd_kernel<128, 8, true>" : "trn::attn_fwd_kernel<128, 4, true>";
    return wide ? "trn::attn_fwd_kernel<64, 8, true>" : "trn::attn_fwd_kernel<64, 4, true>";
}

extern "C" int trn_attn_fwd_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                void* stream) {
    return trn_attn_fwd_ws_f16(d, q, k, v, o, lse, gamma_q, noise, lse_pert, nullptr, 0, stream);
}

extern "C" int trn_attn_fwd_ws_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                   float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
    return trn::attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, workspace, workspace_bytes, nullptr, nullptr, stream);
}

extern "C" int trn_attn_colstats_f16(const trn_attn_desc* d, const void* q, const void* k, const float* lse,
                                     const float* noise, float* out_sum, float* out_sumsq, void* stream);

extern "C" int trn_attn_fwd_probs_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                      float* lse, const float* noise, float* lse_pert,
                                      float* out_probs, float* out_sum, void* stream) {
    using namespace trn;
    if (!d || !out_probs) return TRN_E_NULL;
    if (d->seq_q > 32) return TRN_E_UNSUPPORTED;     // the un-reduced matrix is a decode-shape output
    if (d->q_norm) return TRN_E_UNSUPPORTED;
    return attn_forward(d, q, k, v, o, lse, nullptr, noise, lse_pert, nullptr, 0, out_sum, nullptr, stream, out_probs);
}

extern "C" int trn_attn_fwd_stats_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                      float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                      float* out_sum, float* out_sumsq, void* stream) {
    using namespace trn;
    if (!d) return TRN_E_NULL;
    if (!out_sum && !out_sumsq) return TRN_E_NULL;
    if (d->q_norm) return TRN_E_UNSUPPORTED;     // the statistics pass takes the queries as given
    // a handful of queries per head: the statistics are a second sweep inside the same kernel
    if (d->seq_q <= 32) return attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, nullptr, 0, out_sum, out_sumsq, stream);
    // otherwise two launches; the second needs the first one's row normalisers
    float* rows = noise ? lse_pert : lse;
    if (!rows) return TRN_E_NULL;
    const int st = attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, nullptr, 0, nullptr, nullptr, stream);
    if (st != TRN_OK) return st;
    return trn_attn_colstats_f16(d, q, k, rows, noise, out_sum, out_sumsq, stream);
}

// Where two launches (keys split over workgroups, then the statistics over all keys at once) beat the single launch
// whose two sweeps run with one workgroup per head and column share.  Measured, 16 queries per head, microseconds one
// launch / two launches, RoCo (KeyFormer): 8 heads of 128: 27 / 35 (33 / 30) at 4 k keys, 47 / 38 (59 / 39) at 8 k, 163 /
// 78 (209 / 77) at 32 k; 16 heads of 64: 24 / 30 (33 / 31) at 4 k, 44 / 41 (60 / 42) at 8 k; 16 heads of 128: 48 / 55
// (61 / 55) at 8 k, 87 / 81 (112 / 79) at 16 k; 32 heads of 128: 48 / 65 (59 / 64) at 8 k, 165 / 189 (207 / 183) at 32 k;
// 48 heads: the single launch at every length.  The crossover follows the work per key, heads x head_dim: up to 2048 of
// it, from 8 keys per unit (1024: 8192 keys, 2048: 16384), never below 4096 keys.
extern "C" int64_t trn_attn_stats_workspace_bytes(const trn_attn_desc* d) {
    const int64_t need = trn_attn_workspace_bytes(d);
    if (need == 0) return 0;
    const int64_t per_key = (int64_t)d->batch * d->n_q_heads * d->head_dim;
    return per_key <= 2048 && d->seq_kv >= (8 * per_key > 4096 ? 8 * per_key : 4096) ? need : 0;
}

extern "C" int trn_attn_fwd_stats_ws_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                         float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                         float* out_sum, float* out_sumsq, void* workspace, int64_t workspace_bytes,
                                         void* stream) {
    using namespace trn;
    if (!d) return TRN_E_NULL;
    if (!out_sum && !out_sumsq) return TRN_E_NULL;
    if (d->q_norm) return TRN_E_UNSUPPORTED;
    if (workspace && ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0 || workspace_bytes < 0)) return TRN_E_ALIGN;
    // Few queries and few heads on a long cache: the keys are split over workgroups (which needs the workspace), and
    // the statistics, which need the merged row normalisers, follow as a launch of their own over all keys at once --
    // if the caller gave the buffer that carries the normalisers.  Everything else runs as trn_attn_fwd_stats_f16.
    const int64_t need = trn_attn_stats_workspace_bytes(d);
    float* rows = noise ? lse_pert : lse;
    if (workspace && need > 0 && workspace_bytes >= need && rows) {
        const int st = attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, workspace, workspace_bytes, nullptr, nullptr, stream);
        if (st != TRN_OK) return st;
        return trn_attn_colstats_f16(d, q, k, rows, noise, out_sum, out_sumsq, stream);
    }
    return trn_attn_fwd_stats_f16(d, q, k, v, o, lse, gamma_q, noise, lse_pert, out_sum, out_sumsq, stream);
}

extern "C" int trn_attn_fwd_stats_half_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                           float* lse, const void* gamma_q, const void* noise, float* lse_pert,
                                           void* out_sum, void* out_sumsq, void* stream) {
    using namespace trn;
    if (!d) return TRN_E_NULL;
    if (!out_sum && !out_sumsq) return TRN_E_NULL;
    if (d->q_norm || d->seq_q > 32) return TRN_E_UNSUPPORTED;
    return attn_forward(d, q, k, v, o, lse, gamma_q, static_cast<const float*>(noise), lse_pert, nullptr, 0,
                        static_cast<float*>(out_sum), static_cast<float*>(out_sumsq), stream, nullptr, true);
}

int trn::attn_forward(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o, float* lse,
                             const void* gamma_q, const float* noise, float* lse_pert, void* workspace,
                             int64_t workspace_bytes, float* col_sum, float* col_sumsq, void* stream, float* probs,
                             bool io16) {
    if (workspace && ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0 || workspace_bytes < 0)) return TRN_E_ALIGN;
    if (!d || !q || !k || !v || !o) return TRN_E_NULL;
    if (noise && !lse_pert) return TRN_E_NULL;
    int st = validate_attn(d, true);
    if (st != TRN_OK) return st;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || (gamma_q && !aligned16(gamma_q)))
        return TRN_E_ALIGN;
    if (noise) {
        if (!(d->tau > 0.f)) return TRN_E_UNSUPPORTED;
        if (d->noise_stride_s < d->seq_kv) return TRN_E_STRIDE;
        // one head's noise is addressed with 32-bit byte offsets
        if ((int64_t)d->seq_q * d->noise_stride_s * 4 + 1024 > 0x7fffffffLL) return TRN_E_UNSUPPORTED;
        if (io16) {     // fp16 noise is fetched 8 bytes at a time
            if ((reinterpret_cast<uintptr_t>(noise) & 7u) || (d->noise_stride_s & 3) || (d->noise_stride_h & 3) || (d->noise_stride_b & 3))
                return TRN_E_ALIGN;
        } else if (!aligned16(noise) || !pitch16(d->noise_stride_s, 4) || !pitch16(d->noise_stride_h, 4) ||
                   !pitch16(d->noise_stride_b, 4))
            return TRN_E_ALIGN;
    }
    if (io16 && d->seq_q > 32) return TRN_E_UNSUPPORTED;     // fp16 noise and statistics: the decode kernel only
    AttnArgs a;
    a.q = (const half_t*)q; a.k = (const half_t*)k; a.v = (const half_t*)v; a.o = (half_t*)o;
    a.lse = lse; a.gamma_q = (const half_t*)gamma_q; a.noise = noise; a.lse_pert = lse_pert;
    a.B = d->batch; a.Hq = d->n_q_heads; a.Hkv = d->n_kv_heads; a.Sq = d->seq_q; a.Skv = d->seq_kv;
    a.n_qtiles = 0;   // set per tile shape at launch
    a.qb = d->q_stride_b; a.qh = d->q_stride_h; a.qs = d->q_stride_s;
    a.kb = d->k_stride_b; a.kh = d->k_stride_h; a.ks = d->k_stride_s;
    a.vb = d->v_stride_b; a.vh = d->v_stride_h; a.vs = d->v_stride_s;
    a.ob = d->o_stride_b; a.oh = d->o_stride_h; a.os = d->o_stride_s;
    a.nb = d->noise_stride_b; a.nh = d->noise_stride_h; a.ns = d->noise_stride_s;
    a.c1 = d->scale * kLog2e;
    const float tau = noise ? d->tau : 1.f;
    a.c2 = d->scale * kLog2e / tau; a.c3 = kLog2e / tau;
    a.q_eps = d->q_norm_eps; a.causal = d->causal ? 1 : 0; a.q_norm = d->q_norm ? 1 : 0;
    a.n_split = 1; a.ws = nullptr; a.col_sum = col_sum; a.col_sumsq = col_sumsq; a.probs = probs; a.io16 = io16 ? 1 : 0;
    // K/V tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base
    // (with room for the blocks the pipelines request past the end, which must stay representable to read as zeros)
    if (((int64_t)d->seq_kv + 2048) * d->k_stride_s * 2 > 0x7fffffffLL || ((int64_t)d->seq_kv + 2048) * d->v_stride_s * 2 > 0x7fffffffLL)
        return TRN_E_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    // a handful of queries per head (decode): one workgroup per head, its waves split the keys
    if (d->seq_q <= 32)
        return launch_attn_decode(a, d->head_dim, workspace, workspace_bytes, s) == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
    // Without score perturbation: the 16x16x32 kernel, in the workgroup shape its launcher's rule picks.
    if (!noise)
        return launch_attn_fwd16(a, d->head_dim, attn_fwd16_shape(d->batch, d->n_q_heads, d->seq_q, d->head_dim, d->causal != 0), s) == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
    // With it: 8 waves x 32 queries per workgroup (one workgroup per CU; each K/V stage is fetched from L2 once per
    // 256 queries) when that still fills the chip -- one workgroup per CU for unmasked attention, two rounds under a
    // causal mask, where workgroups differ in length; otherwise 4 waves x 32 (two workgroups per CU).
    const bool wide = noise_kernel_wide(d);
#define TRN_LAUNCH(D_, NW_) launch_fwd<D_, NW_, true>(a, s)
    if (d->head_dim == 128) e = wide ? TRN_LAUNCH(128, 8) : TRN_LAUNCH(128, 4);
    else e = wide ? TRN_LAUNCH(64, 8) : TRN_LAUNCH(64, 4);
#undef TRN_LAUNCH
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
