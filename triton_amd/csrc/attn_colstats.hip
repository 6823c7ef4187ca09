// Per-key column statistics of the attention probabilities (KeyFormer key scores, RoCo sum / sum of squares).
//
//     p_ij = exp(t_ij - lse_i);   out_sum[j] = sum_i p_ij;   out_sumsq[j] = sum_i p_ij^2
// with t = scale*QK^T (RoCo) or (scale*QK^T + noise)/tau (KeyFormer) and lse_i the matching row normaliser
// produced by the forward kernel.  A column sum needs the FINAL row normalisers, so this is a second pass
// that recomputes QK^T on MFMA instead of storing an S x S matrix.
//
// Column-owner design: a workgroup owns 128 keys (32 per wave) of one (batch, head) and walks over the query
// tiles that can see them.  As in the forward kernel the product is formed transposed, S^T[key][query], with
// the wave's K rows held in registers as the A operand for the whole walk and Q tiles staged through LDS as
// the B operand.  Lane l then holds 16 keys x ONE query, so the per-query normaliser is one scalar per lane,
// and each lane accumulates its 16 per-key partial sums in registers across all query tiles; the sum over
// the 32 queries held by different lanes is done once at the end.  No atomics: results are deterministic.
//
// Q tiles of 64 queries go straight from global memory into a ring of three LDS stages (buffer_load ... lds,
// XOR-swizzled rows), requested two tiles ahead, one barrier per tile.  What the VALU needs per tile besides the scores -- the row
// normalisers and, for KeyFormer, the wave's 64 x 32 block of fp32 noise, which is the HBM stream that bounds
// that variant -- is loaded into registers one to two tiles ahead (a block's registers are refilled as soon as it
// has been consumed), so that a CU has 64 - 128 KB of noise in flight.  All of these loads are buffer loads with out-of-range zero fill and are issued unconditionally
// in a fixed order: the wait for a Q stage counts the loads issued behind it.  Masks (causal diagonal, ragged
// ends) are evaluated only in the blocks that need them (a wave-uniform test).
#include <type_traits>
#include "common.h"

namespace trn {

int validate_attn(const trn_attn_desc* d, bool need_v);

struct ColArgs {
    const half_t* q; const half_t* k; const float* lse; const float* noise;
    float* out_sum; float* out_sumsq;
    int B, Hq, Hkv, Sq, Skv, n_kvtiles;
    int64_t qb, qh, qs, kb, kh, ks, nb, nh, ns;
    float c1;   // log2-domain multiplier of the raw score: scale*log2e (RoCo) or scale*log2e/tau (KeyFormer)
    float c3;   // log2e/tau multiplier of the noise
    int causal;
    int pair;       // (no-noise kernel) a workgroup takes key tiles i and n-1-i
    int mean_std;   // write the per-key mean and population standard deviation over the queries that see the key
                    // (into out_sum / out_sumsq) instead of the two sums
};

constexpr int CBN = 128;  // keys per workgroup
[[maybe_unused]] constexpr int CBM = 64;   // queries per staged tile

// SQ: the sums of squares are wanted too (RoCo); without them (KeyFormer) their accumulators and one of the five
// VALU operations per score are not compiled in.
template <int D, bool NOISE, bool SQ>
__global__ __launch_bounds__(256, NOISE ? 2 : 3) void attn_colstats_kernel(const ColArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    constexpr int NKS = D / 16;
    constexpr int CPR = D / 8;                 // 16-byte chunks per Q row
    constexpr int RPI = 64 / CPR;              // stage rows covered by one wave-wide 1 KB load
    constexpr int NI = CBM / (RPI * 4);        // such loads per wave per stage
    __shared__ __attribute__((aligned(1024))) half_t Qs0[CBM * D];
    __shared__ __attribute__((aligned(1024))) half_t Qs1[CBM * D];
    __shared__ __attribute__((aligned(1024))) half_t Qs2[CBM * D];
    // KeyFormer: the wave's 32 x 32 block of noise is fetched with whole 128-byte row pieces per 8 lanes (a load
    // instruction then touches 8 cache lines, not 32) and turned into the accumulator layout through this array
    __shared__ __attribute__((aligned(1024))) float Ns[NOISE ? 4 * 1024 : 4];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int BH = a.B * a.Hq;
    const int kt = (int)(blockIdx.x / BH);             // key tile 0 sees the most queries: heaviest first
    const int j = blockIdx.x % BH;
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;
    const int off = a.Skv - a.Sq;
    const int kv0 = kt * CBN;
    const int wkey0 = kv0 + wave * 32;                 // this wave's 32 keys

    // K rows of this wave as MFMA A-operands, resident for the whole walk
    half8_t kA[NKS];
    {
        const int key = min(wkey0 + c, a.Skv - 1);
        const half_t* kp = a.k + b * a.kb + kvh * a.kh + (int64_t)key * a.ks + 8 * h;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) kA[ks] = *reinterpret_cast<const half8_t*>(kp + ks * 16);
    }

    float s1[16], s2[SQ ? 16 : 1];
#pragma unroll
    for (int r = 0; r < 16; ++r) { s1[r] = 0.f; if constexpr (SQ) s2[r] = 0.f; }

    // ---- Q stages: direct global -> LDS; queries past the end read as zeros
    const __amdgpu_buffer_rsrc_t qrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.q + b * a.qb + head * a.qh), 0, (int)(((int64_t)(a.Sq - 1) * a.qs + D) * 2), 0x00020000);
    const int st_row = wave * RPI + lane / CPR;
    const int st_chunk = (lane % CPR) ^ swz<D>(st_row);
    const int qvo = (int)(st_row * a.qs * 2) + st_chunk * 16;
    const int qrow_bytes = (int)(RPI * a.qs * 2), qtile_bytes = (int)(CBM * a.qs * 2);
#define TRN_FETCH_Q(t_, dst_) fetch_tile<NI, D, 4>(qrs, &dst_[wave * RPI * D], qvo, (t_) * qtile_bytes, qrow_bytes)
    int qoff[NKS];       // B-operand read: row c (+32 for the second block), logical chunk 2*ks + h
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qoff[ks] = c * D + (((2 * ks + h) ^ swz<D>(c)) << 3);

    // ---- per-tile register prefetch: row normalisers and noise of the tile's two 32-query blocks
    const __amdgpu_buffer_rsrc_t lrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.lse + ((int64_t)b * a.Hq + head) * a.Sq), 0, a.Sq * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t nrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(NOISE ? a.noise + b * a.nb + head * a.nh : a.lse), 0,
        NOISE ? (int)(((int64_t)(a.Sq - 1) * a.ns + a.Skv) * 4) : 0, 0x00020000);
    // load i of a block covers its query rows 8i .. 8i+7: lane -> row 8i + lane/8, keys 4*(lane%8) .. +3
    const int nvo = NOISE ? (int)(((lane >> 3) * a.ns + wkey0 + 4 * (lane & 7)) * 4) : 0;
    const int nrow8 = NOISE ? (int)(8 * a.ns * 4) : 0;
    // transposer: the 16-byte chunk q of row r sits at chunk r*8 + (q ^ ((r/2) % 8)); written as loaded, read as
    // row c, chunks 2*r4 + h (both conflict-free)
    float* nsw = Ns + (NOISE ? wave * 1024 : 0);
    int ns_wr[4], ns_rd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = 8 * i + (lane >> 3);
        ns_wr[i] = (r * 8 + ((lane & 7) ^ ((r >> 1) & 7))) * 4;
        ns_rd[i] = (c * 8 + ((2 * i + h) ^ ((c >> 1) & 7))) * 4;
    }
    // Two register buffers, used by even and odd tiles in turn.  A block's half of a buffer is refilled, for the tile
    // after next, as soon as that block has been consumed, so between one and two tiles of noise (8 - 16 KB per
    // wave) are in flight at any time.
    struct Pre { float lse[2]; float4_t g[2][4]; };
    Pre pa, pb;
    auto prefetch = [&](int t, int qb, Pre& p) __attribute__((always_inline)) {
        p.lse[qb] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(lrs, c * 4, (t * CBM + qb * 32) * 4, 0));
        if constexpr (NOISE) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
                p.g[qb][r4] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                    nrs, nvo + r4 * nrow8, (int)((t * CBM + qb * 32) * a.ns * 4), 0));
        }
    };

    const int first_q = a.causal ? max(0, kv0 - off) : 0;   // earlier queries see none of this tile's keys
    const int t0 = first_q / CBM, nt = (a.Sq + CBM - 1) / CBM;

    // The VALU part of a 32-query block.  Masked and plain blocks are separate loops (one wave-uniform branch
    // per block) so that the plain one is 4 instructions per score: fma, exp2, add, fma.
    auto softmax_sums = [&](const float16_t& acc, int qfirst, float lse, const float4_t (&gl)[4]) __attribute__((always_inline)) {
        const float lse2 = lse * kLog2e;
        float4_t gq[4];
        if constexpr (NOISE) {       // (LDS operations of one wave execute in order: no barrier between the two)
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<float4_t*>(&nsw[ns_wr[i]]) = gl[i];
#pragma unroll
            for (int i = 0; i < 4; ++i) gq[i] = *reinterpret_cast<const float4_t*>(&nsw[ns_rd[i]]);
        }
        const bool masked = (qfirst + 31 >= a.Sq) || (wkey0 + 31 >= a.Skv) || (a.causal && wkey0 + 31 > qfirst + off);
        if (masked) {
            // last key this lane's query may count, as an offset from the lane's first key (-1: none)
            const int qrow = qfirst + c;
            const int last = qrow < a.Sq ? min(a.causal ? qrow + off : a.Skv - 1, a.Skv - 1) - (wkey0 + 4 * h) : -1;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float t = __builtin_fmaf(acc[r], a.c1, -lse2);
                if constexpr (NOISE) t = __builtin_fmaf(gq[r / 4][r % 4], a.c3, t);
                const float p = (8 * (r / 4) + (r % 4) <= last) ? fast_exp2(t) : 0.f;
                s1[r] += p;
                if constexpr (SQ) s2[r] = __builtin_fmaf(p, p, s2[r]);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float t = __builtin_fmaf(acc[r], a.c1, -lse2);
                if constexpr (NOISE) t = __builtin_fmaf(gq[r / 4][r % 4], a.c3, t);
                const float p = fast_exp2(t);
                s1[r] += p;
                if constexpr (SQ) s2[r] = __builtin_fmaf(p, p, s2[r]);
            }
        }
    };
    // The two 32-query blocks of a tile.  Each block's eight score MFMAs accumulate into one register block (a
    // dependent chain); all operands of a chain are in registers before it starts, and the second block's are
    // read while the first chain runs.
    auto blocks = [&](const half_t* Qc, int t, Pre& pc) __attribute__((always_inline)) {
        const int q0 = t * CBM;
        // (causal) none of a block's queries sees any of this wave's keys: skip it
        const bool live0 = !(a.causal && q0 + 31 + off < wkey0), live1 = !(a.causal && q0 + 63 + off < wkey0);
        float16_t acc0, acc1;
        if (live1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
            half8_t qa[NKS];
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) qa[ks] = *reinterpret_cast<const half8_t*>(&Qc[qoff[ks]]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                acc0 = mfma32(kA[ks], qa[ks], acc0);
                qa[ks] = *reinterpret_cast<const half8_t*>(&Qc[32 * D + qoff[ks]]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) acc1 = mfma32(kA[ks], qa[ks], acc1);
            __builtin_amdgcn_sched_barrier(0);
            if (live0) softmax_sums(acc0, q0, pc.lse[0], pc.g[0]);
        }
        prefetch(t + 2, 0, pc);              // (unconditional, like every load of the loop: see below)
        if (live1) softmax_sums(acc1, q0 + 32, pc.lse[1], pc.g[1]);
        prefetch(t + 2, 1, pc);
    };
    // Tile t reads stage t % 3; the stage of tile t+2 is requested as soon as the barrier shows that everybody has
    // left tile t-1 (its previous tenant), so a Q stage has two tile times to arrive from L2.  Tile t's stage has
    // landed once this wave's own share has, and the others' too.  Behind this wave's share of stage t these have
    // been issued, in this order: the register prefetch of tile t (during tile t-2), stage t+1, the register
    // prefetch of tile t+1 (during tile t-1): NI + 4 requests (+ 16 with noise).  All of them are issued
    // unconditionally (past the last tile everything reads as zeros, the stages into one nobody uses): the compiler
    // sizes its own waits for prefetched registers by the loads it KNOWS follow them, and a conditional load counts
    // as absent, which would make every use of a prefetched value drain the refills too.
    auto tile = [&](int t, const half_t* Qc, half_t* Qf, Pre& pc) __attribute__((always_inline)) {
        constexpr int kBehind = NI + 4 + (NOISE ? 16 : 0);
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kBehind & 15) | ((kBehind >> 4) << 14));
        __builtin_amdgcn_s_barrier();        // (a bare barrier: nothing else in flight needs draining)
        __builtin_amdgcn_sched_barrier(0);
        TRN_FETCH_Q(t + 2, Qf);
        __builtin_amdgcn_sched_barrier(0);
        blocks(Qc, t, pc);
    };
    // the same order of requests as in the loop, so that the count above holds from the first tile on
    TRN_FETCH_Q(t0, Qs0);
    prefetch(t0, 0, pa); prefetch(t0, 1, pa);
    TRN_FETCH_Q(t0 + 1, Qs1);
    prefetch(t0 + 1, 0, pb); prefetch(t0 + 1, 1, pb);
    // Pin the arrival of the K rows here, ahead of the loop.  Left to the first MFMA that reads them, the wait the
    // compiler inserts sits inside the loop body and, being conservative across the back edge, drains the stage and
    // prefetch loads of every iteration.
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) asm volatile("" ::"v"(kA[ks]));
    for (int t = t0; t < nt; t += 6) {       // three stages x two register buffers
        tile(t, Qs0, Qs2, pa);
        if (t + 1 < nt) tile(t + 1, Qs1, Qs0, pb);
        if (t + 2 < nt) tile(t + 2, Qs2, Qs1, pa);
        if (t + 3 < nt) tile(t + 3, Qs0, Qs2, pb);
        if (t + 4 < nt) tile(t + 4, Qs1, Qs0, pa);
        if (t + 5 < nt) tile(t + 5, Qs2, Qs1, pb);
    }
#undef TRN_FETCH_Q

    // sum over the 32 queries held by lanes c = 0..31 (same h), then lane c == 0 of each half writes
    const int64_t obase = ((int64_t)b * a.Hq + head) * a.Skv;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        float x = s1[r], y = SQ ? s2[SQ ? r : 0] : 0.f;
#pragma unroll
        for (int msk = 1; msk < 32; msk <<= 1) { x += __shfl_xor(x, msk, 64); if constexpr (SQ) y += __shfl_xor(y, msk, 64); }
        const int key = wkey0 + 8 * (r / 4) + 4 * h + (r % 4);
        if (SQ && a.mean_std) {
            // n = queries that see this key: all of them, or under a causal mask those from key - (Skv - Sq) on
            const float n = (float)(a.causal ? a.Sq - max(0, key - (a.Skv - a.Sq)) : a.Sq);
            const float mean = x / n;
            // E p^2 - mean^2 as (y - x mean) / n, the product fused.  The difference is known to about 1e-7 of E p^2, its
            // root to 3e-4 of the column's root mean square: a key seen by a single query, whose spread is zero by
            // definition, would come back as that rounding residue, so it is set.
            y = n > 1.5f ? __builtin_sqrtf(fmaxf(0.f, __builtin_fmaf(-x, mean, y) / n)) : 0.f;
            x = mean;
        }
        if (c == 0 && key < a.Skv) {
            if (a.out_sum) a.out_sum[obase + key] = x;
            if (SQ && a.out_sumsq) a.out_sumsq[obase + key] = y;
        }
    }
#endif
}

// Without noise (RoCo, plain column sums) the pass is bound by the vector unit -- four instructions per score (fma,
// exp2, add, fma) against one 32-clock MFMA per 128 scores -- so this variant is arranged for it:
//   * the score MFMAs of tile t+1 are issued between the VALU work of tile t, two scores' worth behind each MFMA
//     (a wave overlaps its own matrix and vector work instead of relying on a neighbour being in the other phase),
//     and the chains of the tile's two 32-query blocks alternate: one chain of MFMAs that each wait for the one
//     before ran the matrix pipe at 40 % even with nothing else to do;
//   * query tiles whose blocks need no mask for any of the workgroup's waves run in a loop of their own whose VALU
//     part has no select and no branch, so the 32 running sums stay in their registers; the few tiles at the
//     causal diagonal and at ragged ends run the same code with a per-score select (blocks wholly before a wave's
//     keys are simply masked away);
//   * the row normalisers ride along with the Q stage (one 256-byte global->LDS load per wave and tile) instead of
//     a register prefetch of their own;
//   * under a causal mask a workgroup takes a heavy and a light key tile in turn, so that all have equal work.
// Ring of four Q stages relative to the first tile.  Tile t+1 is multiplied during step t (the VALU work of tile
// t); at the barrier that opens step t every wave is done with stage t, which is refilled there with tile t+4 --
// three steps before its use.
template <int D, bool SQ>
__global__ __launch_bounds__(256, 2) void attn_colstats_plain_kernel(const ColArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    constexpr int NKS = D / 16;
    constexpr int CPR = D / 8;                 // 16-byte chunks per Q row
    constexpr int RPI = 64 / CPR;              // stage rows covered by one wave-wide 1 KB load
    constexpr int NI = CBM / (RPI * 4);        // such loads per wave per stage
    constexpr int NM = 2 * NKS;                // MFMAs per tile and wave
    constexpr int SPM = 32 / NM;               // scores whose VALU work follows each MFMA
    // One array per stage: the compiler orders LDS reads after outstanding global->LDS loads that may alias them,
    // and only distinct variables are provably disjoint.
    __shared__ __attribute__((aligned(1024))) half_t Qs0[CBM * D];
    __shared__ __attribute__((aligned(1024))) half_t Qs1[CBM * D];
    __shared__ __attribute__((aligned(1024))) half_t Qs2[CBM * D];
    __shared__ __attribute__((aligned(1024))) half_t Qs3[CBM * D];
    __shared__ __attribute__((aligned(256))) float Ls0[4 * CBM];     // each wave keeps its own copy of a tile's 64 normalisers
    __shared__ __attribute__((aligned(256))) float Ls1[4 * CBM];
    __shared__ __attribute__((aligned(256))) float Ls2[4 * CBM];
    __shared__ __attribute__((aligned(256))) float Ls3[4 * CBM];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int BH = a.B * a.Hq;
    const int pidx = (int)(blockIdx.x / BH);
    const int j = blockIdx.x % BH;
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;
    const int off = a.Skv - a.Sq;

    // ---- stages: Q rows and normalisers, direct global -> LDS; queries past the end read as zeros
    const __amdgpu_buffer_rsrc_t qrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.q + b * a.qb + head * a.qh), 0, (int)(((int64_t)(a.Sq - 1) * a.qs + D) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t lrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.lse + ((int64_t)b * a.Hq + head) * a.Sq), 0, a.Sq * 4, 0x00020000);
    const int st_row = wave * RPI + lane / CPR;
    const int st_chunk = (lane % CPR) ^ swz<D>(st_row);
    const int qvo = (int)(st_row * a.qs * 2) + st_chunk * 16;
    const int qrow_bytes = (int)(RPI * a.qs * 2), qtile_bytes = (int)(CBM * a.qs * 2);
#define TRN_FETCH_QL(t_, qd_, ld_)                                                                            \
    do {                                                                                                      \
        fetch_tile<NI, D, 4>(qrs, &qd_[wave * RPI * D], qvo, (t_) * qtile_bytes, qrow_bytes);                 \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                             \
            lrs, (__attribute__((address_space(3))) void*)(&ld_[wave * CBM]), 4, lane * 4, (t_) * CBM * 4, 0, 0); \
    } while (0)
    int qoff[NKS];       // B-operand read: row c (+32 for the second block), logical chunk 2*ks + h
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qoff[ks] = c * D + (((2 * ks + h) ^ swz<D>(c)) << 3);
    const int nt = (a.Sq + CBM - 1) / CBM;

    // Under a causal mask key tile kt is seen by the query tiles from its own position on, so the work falls
    // linearly with kt: a workgroup then takes tile pidx and, after it, tile n-1-pidx (a.pair), and every workgroup
    // has the same amount to do.
    for (int pass = 0; pass < 2; ++pass) {
    int kt = pidx;
    if (pass == 1) {
        kt = a.n_kvtiles - 1 - pidx;
        if (!a.pair || kt <= pidx) break;
        __builtin_amdgcn_s_barrier();          // everybody has left the stages of the first tile's walk
    }
    const int kv0 = kt * CBN;
    const int wkey0 = kv0 + wave * 32;                 // this wave's 32 keys

    // K rows of this wave as MFMA A-operands, resident for the whole walk
    half8_t kA[NKS];
    {
        const int key = min(wkey0 + c, a.Skv - 1);
        const half_t* kp = a.k + b * a.kb + kvh * a.kh + (int64_t)key * a.ks + 8 * h;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) kA[ks] = *reinterpret_cast<const half8_t*>(kp + ks * 16);
    }
    float s1[16], s2[SQ ? 16 : 1];
#pragma unroll
    for (int r = 0; r < 16; ++r) { s1[r] = 0.f; if constexpr (SQ) s2[r] = 0.f; }

    const int first_q = a.causal ? max(0, kv0 - off) : 0;   // earlier queries see none of this tile's keys
    const int t0 = first_q / CBM;
    // Tiles [tg, tp) need no mask for any wave of the workgroup: whole tiles inside the queries, all 128 keys inside
    // the keys and, under a causal mask, visible to the tile's first query.
    int tg = t0, tp = t0;
    if (kv0 + CBN <= a.Skv) {
        if (a.causal) tg = max(t0, (kv0 + CBN - 1 - off + CBM - 1) / CBM);
        tp = a.Sq / CBM;
    }

    // The MFMAs of one tile (Q rows at Qn; the chains of its two blocks alternate), each followed by SPM scores'
    // worth of the VALU work of the tile before it (scores ac0 / ac1, first query qfirst, normalisers l0 / l1).
    auto tile_step = [&](auto maymask_tag, auto valu_tag, const float16_t& ac0, const float16_t& ac1, int qfirst,
                         float l0, float l1, float16_t& an0, float16_t& an1, const half_t* Qn) __attribute__((always_inline)) {
        constexpr bool MAYMASK = decltype(maymask_tag)::value, VALU = decltype(valu_tag)::value;
        const float lse2[2] = {l0 * kLog2e, l1 * kLog2e};
        // last key this lane's query may count, as an offset from the lane's first key (-1: none)
        int last[2] = {32, 32};
        if constexpr (MAYMASK && VALU) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const int qrow = qfirst + 32 * blk + c;
                last[blk] = qrow < a.Sq ? min(a.causal ? qrow + off : a.Skv - 1, a.Skv - 1) - (wkey0 + 4 * h) : -1;
            }
        }
        constexpr int QW = 4;                        // Q operands in flight ahead of their MFMAs
        half8_t qa[QW];
#pragma unroll
        for (int i = 0; i < QW; ++i) qa[i] = *reinterpret_cast<const half8_t*>(&Qn[(i & 1) * 32 * D + qoff[i >> 1]]);
        const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            const int ks = i >> 1;
            if (i & 1) an1 = mfma32(kA[ks], qa[i % QW], ks == 0 ? zero : an1);
            else an0 = mfma32(kA[ks], qa[i % QW], ks == 0 ? zero : an0);
            if (i + QW < NM) qa[i % QW] = *reinterpret_cast<const half8_t*>(&Qn[((i + QW) & 1) * 32 * D + qoff[(i + QW) >> 1]]);
            if constexpr (VALU) {
#pragma unroll
                for (int sidx = i * SPM; sidx < (i + 1) * SPM; ++sidx) {
                    const int blk = sidx >> 4, r = sidx & 15;
                    const float t = __builtin_fmaf(blk ? ac1[r] : ac0[r], a.c1, -lse2[blk]);
                    float p = fast_exp2(t);
                    if constexpr (MAYMASK) p = (8 * (r / 4) + (r % 4) <= last[blk]) ? p : 0.f;
                    s1[r] += p;
                    if constexpr (SQ) s2[r] = __builtin_fmaf(p, p, s2[r]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    float16_t accA, accB, accC, accD;   // scores of the two 32-query blocks of the tile in hand and of the next one
    float lseA, lseB;                   // the lanes' row normalisers for the tile in hand
    // Step t: Qc / Lc = tile t's stage (everybody is done with it: refilled with tile t+4), Qn / Ln = tile t+1's.
    auto step = [&](auto maymask_tag, int t, half_t* Qc, float* Lc, const half_t* Qn, const float* Ln,
                    const float16_t& c0, const float16_t& c1, float16_t& n0, float16_t& n1) __attribute__((always_inline)) {
        // Stage t+1 must have landed: behind this wave's share of it stages t+2 and t+3 have been requested.
        // lgkmcnt(0): this wave's reads of stage t have returned, so the refill cannot overtake them.
        constexpr int kBehind = 2 * (NI + 1);
        __builtin_amdgcn_s_waitcnt(0x0070 | (kBehind & 15) | ((kBehind >> 4) << 14));
        __builtin_amdgcn_s_barrier();        // (a bare barrier: the loads in flight must stay in flight)
        __builtin_amdgcn_sched_barrier(0);
        TRN_FETCH_QL(t + 4, Qc, Lc);         // (unconditional: past the last tile everything reads as zeros)
        __builtin_amdgcn_sched_barrier(0);
        const float l0 = lseA, l1 = lseB;
        lseA = Ln[wave * CBM + c]; lseB = Ln[wave * CBM + 32 + c];      // the next tile's normalisers
        tile_step(maymask_tag, std::true_type{}, c0, c1, t * CBM, l0, l1, n0, n1, Qn);
    };
    // A turn of the ring: four steps (the accumulator pairs swap roles from step to step).
    auto turn = [&](auto maymask_tag, int t, auto&& last) __attribute__((always_inline)) {
        step(maymask_tag, t, Qs0, Ls0, Qs1, Ls1, accA, accB, accC, accD);
        if (last(t)) return true;
        step(maymask_tag, t + 1, Qs1, Ls1, Qs2, Ls2, accC, accD, accA, accB);
        if (last(t + 1)) return true;
        step(maymask_tag, t + 2, Qs2, Ls2, Qs3, Ls3, accA, accB, accC, accD);
        if (last(t + 2)) return true;
        step(maymask_tag, t + 3, Qs3, Ls3, Qs0, Ls0, accC, accD, accA, accB);
        return last(t + 3);
    };

    // ---- prologue: four stages in flight, the first tile multiplied
    TRN_FETCH_QL(t0, Qs0, Ls0);
    TRN_FETCH_QL(t0 + 1, Qs1, Ls1);
    TRN_FETCH_QL(t0 + 2, Qs2, Ls2);
    TRN_FETCH_QL(t0 + 3, Qs3, Ls3);
    {
        constexpr int kBehind = 3 * (NI + 1);
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kBehind & 15) | ((kBehind >> 4) << 14));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        lseA = Ls0[wave * CBM + c]; lseB = Ls0[wave * CBM + 32 + c];
        tile_step(std::false_type{}, std::false_type{}, accA, accB, 0, 0.f, 0.f, accA, accB, Qs0);
    }
    // Three loops of whole turns: masking code up to the first turn whose four tiles are all plain, the code without
    // masks for the turns of plain tiles, masking code for the rest.  Only the last loop leaves in the middle of a
    // turn; the first may run up to three tiles past the end of the queries (they read as zeros and are masked
    // away).  Every loop is thus entered with the same loads in flight as its own back edge brings -- after a loop
    // that might have ended on another stage, the compiler's own wait before a tile's first LDS read would drain
    // stages still in flight.
    const int n_pre = (min(tg, nt) - t0 + 3) / 4, n_plain = max(0, tp - (t0 + 4 * n_pre)) / 4;
    int t = t0;
    auto never = [&](int) { return false; };
    for (int i = 0; i < n_pre; ++i, t += 4) turn(std::true_type{}, t, never);
    for (int i = 0; i < n_plain; ++i, t += 4) turn(std::false_type{}, t, never);
    for (; t < nt; t += 4)
        if (turn(std::true_type{}, t, [&](int tt) { return tt + 1 >= nt; })) break;
    __builtin_amdgcn_s_waitcnt(0x0f70);     // the refills past the last tile have landed before the stages are given up

    // sum over the 32 queries held by lanes c = 0..31 (same h), then lane c == 0 of each half writes
    const int64_t obase = ((int64_t)b * a.Hq + head) * a.Skv;
#pragma unroll
    for (int r16 = 0; r16 < 16; ++r16) {
        float x = s1[r16], y = SQ ? s2[SQ ? r16 : 0] : 0.f;
#pragma unroll
        for (int msk = 1; msk < 32; msk <<= 1) { x += __shfl_xor(x, msk, 64); if constexpr (SQ) y += __shfl_xor(y, msk, 64); }
        const int key = wkey0 + 8 * (r16 / 4) + 4 * h + (r16 % 4);
        if (SQ && a.mean_std) {
            // n = queries that see this key: all of them, or under a causal mask those from key - (Skv - Sq) on
            const float n = (float)(a.causal ? a.Sq - max(0, key - (a.Skv - a.Sq)) : a.Sq);
            const float mean = x / n;
            // E p^2 - mean^2 as (y - x mean) / n, the product fused.  The difference is known to about 1e-7 of E p^2, its
            // root to 3e-4 of the column's root mean square: a key seen by a single query, whose spread is zero by
            // definition, would come back as that rounding residue, so it is set.
            y = n > 1.5f ? __builtin_sqrtf(fmaxf(0.f, __builtin_fmaf(-x, mean, y) / n)) : 0.f;
            x = mean;
        }
        if (c == 0 && key < a.Skv) {
            if (a.out_sum) a.out_sum[obase + key] = x;
            if (SQ && a.out_sumsq) a.out_sumsq[obase + key] = y;
        }
    }
    }   // pass
#undef TRN_FETCH_QL
#endif
}

template <int D>
static hipError_t launch_col_plain(ColArgs a, hipStream_t s) {
    a.pair = a.causal && a.n_kvtiles > 1;
    const unsigned grid = (unsigned)(a.pair ? (a.n_kvtiles + 1) / 2 : a.n_kvtiles) * a.B * a.Hq;
    if (a.out_sumsq) hipLaunchKernelGGL((attn_colstats_plain_kernel<D, true>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((attn_colstats_plain_kernel<D, false>), dim3(grid), dim3(256), 0, s, a);
    return hipGetLastError();
}

template <int D, bool NOISE>
static hipError_t launch_col(const ColArgs& a, hipStream_t s) {
    const unsigned grid = (unsigned)a.n_kvtiles * a.B * a.Hq;
    if (a.out_sumsq) hipLaunchKernelGGL((attn_colstats_kernel<D, NOISE, true>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((attn_colstats_kernel<D, NOISE, false>), dim3(grid), dim3(256), 0, s, a);
    return hipGetLastError();
}

}  // namespace trn

namespace trn {
static int colstats(const trn_attn_desc* d, const void* q, const void* k, const float* lse, const float* noise,
                    float* out_sum, float* out_sumsq, int mean_std, void* stream);
}

extern "C" int trn_attn_colstats_f16(const trn_attn_desc* d, const void* q, const void* k, const float* lse,
                                     const float* noise, float* out_sum, float* out_sumsq, void* stream) {
    return trn::colstats(d, q, k, lse, noise, out_sum, out_sumsq, 0, stream);
}

extern "C" int trn_attn_colmeanstd_f16(const trn_attn_desc* d, const void* q, const void* k, const float* lse,
                                       float* out_mean, float* out_std, void* stream) {
    if (!out_mean || !out_std) return TRN_E_NULL;
    return trn::colstats(d, q, k, lse, nullptr, out_mean, out_std, 1, stream);
}

static int trn::colstats(const trn_attn_desc* d, const void* q, const void* k, const float* lse, const float* noise,
                         float* out_sum, float* out_sumsq, int mean_std, void* stream) {
    if (!d || !q || !k || !lse) return TRN_E_NULL;
    if (!out_sum && !out_sumsq) return TRN_E_NULL;
    int st = validate_attn(d, false);
    if (st != TRN_OK) return st;
    if (d->q_norm) return TRN_E_UNSUPPORTED;
    if (!aligned16(q) || !aligned16(k)) return TRN_E_ALIGN;
    if (noise) {
        if (!(d->tau > 0.f)) return TRN_E_UNSUPPORTED;
        if (d->noise_stride_s < d->seq_kv) return TRN_E_STRIDE;
        // one head's noise is addressed with 32-bit byte offsets
        if (((int64_t)d->seq_q + 128) * d->noise_stride_s * 4 > 0x7fffffffLL) return TRN_E_UNSUPPORTED;
        if (!aligned16(noise) || !pitch16(d->noise_stride_s, 4) || !pitch16(d->noise_stride_h, 4) ||
            !pitch16(d->noise_stride_b, 4))
            return TRN_E_ALIGN;
    }
    // Q tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base (with room for the tile requested
    // past the end, which must stay representable to read as zeros)
    if (((int64_t)d->seq_q + 128) * d->q_stride_s * 2 > 0x7fffffffLL) return TRN_E_UNSUPPORTED;
    ColArgs a;
    a.q = (const half_t*)q; a.k = (const half_t*)k; a.lse = lse; a.noise = noise;
    a.out_sum = out_sum; a.out_sumsq = out_sumsq;
    a.B = d->batch; a.Hq = d->n_q_heads; a.Hkv = d->n_kv_heads; a.Sq = d->seq_q; a.Skv = d->seq_kv;
    a.n_kvtiles = (d->seq_kv + CBN - 1) / CBN;
    a.qb = d->q_stride_b; a.qh = d->q_stride_h; a.qs = d->q_stride_s;
    a.kb = d->k_stride_b; a.kh = d->k_stride_h; a.ks = d->k_stride_s;
    a.nb = d->noise_stride_b; a.nh = d->noise_stride_h; a.ns = d->noise_stride_s;
    const float tau = noise ? d->tau : 1.f;
    a.c1 = d->scale * kLog2e / tau; a.c3 = kLog2e / tau;
    a.causal = d->causal ? 1 : 0;
    a.mean_std = mean_std; a.pair = 0;
    if ((int64_t)a.n_kvtiles * a.B * a.Hq > 0x7fffffffLL) return TRN_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (d->head_dim == 128) e = noise ? launch_col<128, true>(a, s) : launch_col_plain<128>(a, s);
    else e = noise ? launch_col<64, true>(a, s) : launch_col_plain<64>(a, s);
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
