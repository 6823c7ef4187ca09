// Attention forward for at most 32 queries per head (decode-append: a few new tokens against a long cache).
//
// With so few queries there is one 32-query MFMA block per head and the kernel is a stream of K and V through HBM.
// One workgroup per (batch, head); its eight waves take the 32-key blocks round-robin, each with its own running
// max / normaliser / O^T accumulator, and the eight partial results are merged through LDS at the end (the usual
// log-sum-exp merge).  Formulation and register layouts are those of the prefill kernel: S^T = K Q^T with Q^T
// resident in registers, P^T taken from the S^T accumulator, V^T via the transposing LDS read.  K rows are what the
// A operand wants as they lie in memory, so K goes straight from global memory into registers (one block ahead);
// V goes global -> LDS into the wave's private two-stage ring.  Nothing in the loop is shared between waves, so the
// loop has no barrier; every load is issued unconditionally (blocks past the end read zeros, which are masked) so
// that the waits can be counted.
#include "attn.h"
#include <mutex>

typedef unsigned long long ulong2_t __attribute__((ext_vector_type(2)));

namespace trn {

constexpr int DNW = 8;    // waves per workgroup

// XOR swizzle of the 16-byte chunk index of a V row as wide as this workgroup's share of the head dimension
template <int DV> __device__ __forceinline__ int swzv(int r) {
    if constexpr (DV == 32) return (r >> 1) & 3;          // 4 chunks per 64-byte row
    else return swz<DV>(r);
}

// DS: the head dimension of V and O is shared out over DS workgroups per head (each computes all the scores, from
// all of K, but streams only its DV = D / DS columns of V and writes those columns of O).  One CU pulls 40 - 55 GB/s
// whatever its waves ask for, and with one workgroup per head that rate is what the kernel's time is made of; more
// workgroups per head without anything to hand over between them means fewer bytes through each CU.
// NZ: 0 no score perturbation, 1 fp32 noise, 2 fp16 noise
template <int D, int DS, int NZ>
__global__ __launch_bounds__(DNW * 64, 1) void attn_decode_kernel(const AttnArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    constexpr bool NOISE = NZ != 0, N16 = NZ == 2;
    constexpr int DV = D / DS;    // columns of V / O this workgroup owns
    constexpr int NS = D / 16;    // k-steps of S^T = K Q^T
    constexpr int NSV = DV / 16;  // (2 key halves) x (DV/32) MFMAs of P V
    constexpr int NDB = DV / 32;
    constexpr int CPR = DV / 8;   // 16-byte chunks per V row share
    constexpr int RPI = 64 / CPR; // rows per wave-wide 1 KB load
    constexpr int NI = 32 / RPI;  // such loads per 32-key V block
    // two V stages (each holds the eight waves' private parts), as two arrays: LDS reads are ordered after
    // outstanding global->LDS loads that may alias them, and only distinct variables are provably disjoint
    // (With the whole head dimension of V in one workgroup at head_dim 128 a V stage is 64 KB: one stage then, refilled
    // as soon as its block's P V is issued, so that the K area below still fits.)
    constexpr bool VSINGLE = D == 128 && DS == 1;
    __shared__ __attribute__((aligned(1024))) half_t Vs0[DNW * 32 * DV];
    __shared__ __attribute__((aligned(1024))) half_t Vs1[VSINGLE ? 8 : DNW * 32 * DV];
    __shared__ float st_m[DNW][32], st_l[DNW][32], st_m2[DNW][32], st_l2[DNW][32];
    // K blocks are fetched as whole rows (a wave-wide load = 1 KB of consecutive bytes) and turned into MFMA operands
    // through a wave-private LDS area: a load whose lanes each take 16 bytes of their own row -- the operand layout --
    // is served at 16 bytes per clock (36 GB/s per CU measured), the row-wise one at 64 (130 GB/s).
    constexpr bool KLDS = true;
    constexpr int CPRK = D / 8;       // 16-byte chunks per K row
    constexpr int RPIK = 64 / CPRK;   // K rows per wave-wide load
    __shared__ __attribute__((aligned(1024))) half_t Kt[DNW * 32 * D];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup id -> (batch x head j, key share, column share).  The column shares of a head read the same K: their
    // ids are 8 apart, so that they sit on one XCD (ids are dealt to the 8 XCDs in turn) and share its L2.
    int j, split, dsl;
    if constexpr (DS > 1) {
        const int grp = blockIdx.x / (8 * DS), rem = blockIdx.x % (8 * DS);
        j = grp * 8 + rem % 8; dsl = rem / 8; split = 0;
        if (j >= a.B * a.Hq) return;                    // the last group of eight heads may be short
    } else {
        j = blockIdx.x / a.n_split; split = blockIdx.x % a.n_split; dsl = 0;
    }
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;
    const int off = a.Skv - a.Sq;                       // causal: query i sees keys <= i + off
    const int qrow = c;                                 // this lane's query
    const int qrow_ld = qrow < a.Sq ? qrow : a.Sq - 1;

    // ---- Q^T B-operands: lane holds Q[qrow][ks*16 + 8h .. +7]; optional fused per-head RMSNorm of the row
    half8_t qB[NS];
    {
        const half_t* qp = a.q + b * a.qb + head * a.qh + (int64_t)qrow_ld * a.qs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < NS; ++ks) qB[ks] = *reinterpret_cast<const half8_t*>(qp + ks * 16);
    }
    // ---- K: block rows straight into registers as A operands (lane: key c of the block, columns ks*16 + 8h ..)
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.k + b * a.kb + kvh * a.kh), 0, (int)(((int64_t)(a.Skv - 1) * a.ks + D) * 2), 0x00020000);
    const int kvo = KLDS ? (int)((lane / CPRK) * a.ks * 2) + (lane % CPRK) * 16 : (int)(c * a.ks * 2) + 16 * h;
    const int kblk_bytes = (int)(32 * a.ks * 2), kpiece_bytes = (int)(RPIK * a.ks * 2);
    // With KLDS the registers hold piece i = rows i*RPIK .. +RPIK-1 of the block as they lie in memory (D/16 = NS
    // pieces); k_operands() below turns them into the operands in place.  Without it they are the operands.
    auto fetch_k = [&](int blk, half8_t (&ka)[NS]) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < NS; ++ks) {
            if constexpr (KLDS)
                ka[ks] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(krs, kvo, blk * kblk_bytes + ks * kpiece_bytes, 0));
            else
                ka[ks] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(krs, kvo + ks * 32, blk * kblk_bytes, 0));
        }
    };
    // Rows into the wave's area (chunk j of row r at j ^ swz<D>(r): the write of a piece covers its 1 KB once, and
    // the 32 rows read back at one logical chunk touch every bank once), operands out of it.  LDS operations of one
    // wave execute in order and nobody else touches the area: no barrier.
    auto k_operands = [&](half8_t (&ka)[NS]) __attribute__((always_inline)) {
        if constexpr (KLDS) {
            half_t* kt = Kt + wave * 32 * D;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const int r = i * RPIK + lane / CPRK;
                *reinterpret_cast<half8_t*>(&kt[r * D + (((lane % CPRK) ^ swz<D>(r)) << 3)]) = ka[i];
            }
#pragma unroll
            for (int ks = 0; ks < NS; ++ks)
                ka[ks] = *reinterpret_cast<const half8_t*>(&kt[c * D + (((2 * ks + h) ^ swz<D>(c)) << 3)]);
        }
    };
    // ---- V: block rows global -> LDS, chunk c of row r stored at c ^ swz<D>(r); load n covers rows n*RPI + lane/CPR
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.v + b * a.vb + kvh * a.vh), 0, (int)(((int64_t)(a.Skv - 1) * a.vs + D) * 2), 0x00020000);
    int vvo[NI];
#pragma unroll
    for (int n = 0; n < NI; ++n) {
        const int r = n * RPI + lane / CPR;
        vvo[n] = (int)(r * a.vs * 2) + dsl * DV * 2 + (((lane % CPR) ^ swzv<DV>(r)) << 4);
    }
    const int vblk_bytes = (int)(32 * a.vs * 2);
#define TRN_FETCH_V(blk_, dst_)                                                                                  \
    _Pragma("unroll") for (int n_ = 0; n_ < NI; ++n_) __builtin_amdgcn_raw_ptr_buffer_load_lds(                  \
        vrs, (__attribute__((address_space(3))) void*)(&dst_[wave * 32 * DV + n_ * RPI * DV]), 16, vvo[n_],      \
        (blk_) * vblk_bytes, 0, 0)
    // V^T operand through the transposing read (as in the prefill kernel): rows 4h + (lane%16)/4 [+8] of a 16-key half
    int voff_lo[NDB], voff_hi[NDB];
    {
        const int rl = 4 * h + ((lane & 15) >> 2), rh = rl + 8;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            voff_lo[db] = wave * 32 * DV + rl * DV + (((db * 4 + lc) ^ swzv<DV>(rl)) << 3) + sub;
            voff_hi[db] = wave * 32 * DV + rh * DV + (((db * 4 + lc) ^ swzv<DV>(rh)) << 3) + sub;
        }
    }

    float16_t oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;       // running max (log2 domain, shared by the lane pair) and this lane's partial sum
    float m2 = -INFINITY, l2 = 0.f;     // the same for the perturbed scores (KeyFormer)
    // KeyFormer noise: this lane's query row, the 4 x 4 keys of its accumulator layout per block, one block ahead
    // (fp16 noise: 8-byte pieces of 4 keys, widened as they arrive)
    constexpr int nsz = N16 ? 2 : 4;     // bytes per noise element
    const __amdgpu_buffer_rsrc_t nrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(NOISE ? reinterpret_cast<const char*>(a.noise) + (b * a.nb + head * a.nh) * nsz : nullptr), 0,
        NOISE ? (int)(((int64_t)(a.Sq - 1) * a.ns + (N16 ? (a.Skv + 1) & ~1 : a.Skv)) * nsz) : 0, 0x00020000);
    // (The range check works on whole dwords: with fp16 noise and an odd key count the last row's last key shares its
    // dword with the first half of the row's padding, so the range ends behind that dword -- the rows are padded to
    // 8 bytes -- and keys past the end are discarded by the mask, whatever the padding holds.)
    const int nvo = NOISE ? (int)(((int64_t)qrow_ld * a.ns + 4 * h) * nsz) : 0;
    float4_t g0[4], g1[4];
    auto fetch_noise = [&](int blk, float4_t (&g)[4]) __attribute__((always_inline)) {
        if constexpr (N16) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const half4_t hv = __builtin_bit_cast(half4_t, __builtin_amdgcn_raw_buffer_load_b64(nrs, nvo + r4 * 16, blk * 64, 0));
                g[r4] = float4_t{(float)hv[0], (float)hv[1], (float)hv[2], (float)hv[3]};
            }
        } else {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
                g[r4] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(nrs, nvo + r4 * 32, blk * 128, 0));
        }
    };

    // this workgroup's blocks: a contiguous share of the keys when they are split over several workgroups
    const int nblk_all = (a.Skv + 31) / 32, bps = (nblk_all + a.n_split - 1) / a.n_split;
    const int blk0 = split * bps, nblk = max(0, min(nblk_all, blk0 + bps) - blk0);
    const int nmine = nblk > wave ? (nblk - wave + DNW - 1) / DNW : 0;          // blocks blk0 + wave, + 8, ...
    half8_t ka0[NS], ka1[NS];

    // One 32-key block whose K is in kc and whose V is in stage Vc; the next block's loads go to kn / Vn first.
    auto block = [&](int it, half8_t (&kc)[NS], half8_t (&kn)[NS], const half_t* Vc, half_t* Vn, float4_t (&gc)[4],
                     float4_t (&gn)[4]) __attribute__((always_inline)) {
        const int blk = blk0 + wave + it * DNW, key0 = blk * 32;
        // (with noise the registers are short: K is then single-buffered, refilled as soon as the scores are issued)
        if constexpr (!NOISE) fetch_k(blk + DNW, kn);
        if constexpr (!VSINGLE) {
            // (Vn is the stage the previous block read: the same fence as for the single stage below, so that the order
            // does not hang on where the compiler happens to cut its scheduling regions)
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0)
            TRN_FETCH_V(blk + DNW, Vn);
        }
        if constexpr (NOISE) fetch_noise(blk + DNW, gn);
        float16_t s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        k_operands(kc);
#pragma unroll
        for (int ks = 0; ks < NS; ++ks) s = mfma32(kc[ks], qB[ks], s);
        if constexpr (NOISE) fetch_k(blk + DNW, kc);
        // mask (wave-uniform test), block max, running max, probabilities
        const bool masked = (key0 + 32 > a.Skv) || (a.causal && key0 + 31 > off);
        if (masked) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r / 4) + 4 * h + (r % 4);
                s[r] = (key < a.Skv && (!a.causal || key <= qrow + off)) ? s[r] : -INFINITY;
            }
        }
        if constexpr (NOISE) {          // row normaliser of z = (scale*s + g)/tau in the log2 domain
            float16_t z;
#pragma unroll
            for (int r = 0; r < 16; ++r) z[r] = __builtin_fmaf(gc[r / 4][r % 4], a.c3, s[r] * a.c2);
            if (masked) {               // a select, not arithmetic: what lies past a row's last key (the padding of
                                        // the noise pitch) may be anything, NaN included
#pragma unroll
                for (int r = 0; r < 16; ++r) z[r] = s[r] == -INFINITY ? -INFINITY : z[r];
            }
            const float zmax = fmaxf(m2, half_max(max16(z)));
            if (zmax > -INFINITY) {
                float sum = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += fast_exp2(z[r] - zmax);
                l2 = l2 * fast_exp2(m2 - zmax) + sum;
                m2 = zmax;
            }
        }
        const float smax = half_max(max16(s)) * a.c1;
        const float mnew = fmaxf(m, smax);
        const float mref = mnew == -INFINITY ? 0.f : mnew;     // a row can see nothing of a block
        const float alpha = fast_exp2(m - mref);               // m = -inf: 0
        const half2_t ones = {(half_t)1.f, (half_t)1.f};
        half8_t pB[2];
        l *= alpha;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const half2_t pp = {(half_t)fast_exp2(__builtin_fmaf(s[r], a.c1, -mref)),
                                (half_t)fast_exp2(__builtin_fmaf(s[r + 1], a.c1, -mref))};
            l = __builtin_amdgcn_fdot2(pp, ones, l, false);    // the row sum of exactly the values that multiply V
            pB[r / 8][r % 8] = pp[0]; pB[r / 8][r % 8 + 1] = pp[1];
        }
#pragma unroll
        for (int i = 0; i < NDB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
        m = mnew;
        // this block's V has landed: behind it only the next block's NS + NI (+ 4 noise) requests were issued
        // (one V stage: its refill is issued behind the block's P V, so only K and noise requests are younger)
        constexpr int kBehind = NS + (VSINGLE ? 0 : NI) + (NOISE ? 4 : 0);
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kBehind & 15) | ((kBehind >> 4) << 14));
#pragma unroll
        for (int i = 0; i < NSV; ++i) {
            const half_t* vp = Vc + 16 * (i / NDB) * DV;
            const half4_t lo = lds_read_tr16(vp + voff_lo[i % NDB]);
            const half4_t hi = lds_read_tr16(vp + voff_hi[i % NDB]);
            const half8_t va = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            oacc[i % NDB] = mfma32(va, pB[i / NDB], oacc[i % NDB]);
        }
        // (The refill must not overtake the stage's readers.  The compiler does not order the global->LDS load
        // behind the transposing reads by itself -- left alone it moved the load in front of the last of them -- hence
        // the scheduling fence; the wait makes the reads' return explicit.)
        if constexpr (VSINGLE) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0)
            TRN_FETCH_V(blk + DNW, Vn);
        }
    };
    fetch_k(blk0 + wave, ka0);
    TRN_FETCH_V(blk0 + wave, Vs0);
    if constexpr (NOISE) fetch_noise(blk0 + wave, g0);
    // (the first K / V requests are on their way before Q is waited for: one memory latency instead of two)
    if (a.q_norm) {
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
    // pin the arrival of Q here: left to the first MFMA in the loop, the compiler's wait would sit in the loop body
#pragma unroll
    for (int ks = 0; ks < NS; ++ks) asm volatile("" ::"v"(qB[ks]));
    for (int it = 0; it < nmine; it += 2) {
        if constexpr (NOISE) {
            block(it, ka0, ka0, Vs0, VSINGLE ? Vs0 : Vs1, g0, g1);
            if (it + 1 < nmine) block(it + 1, ka0, ka0, VSINGLE ? Vs0 : Vs1, Vs0, g1, g0);
        } else {
            block(it, ka0, ka1, Vs0, VSINGLE ? Vs0 : Vs1, g0, g1);
            if (it + 1 < nmine) block(it + 1, ka1, ka0, VSINGLE ? Vs0 : Vs1, Vs0, g1, g0);
        }
    }
#undef TRN_FETCH_V

    // ---- merge the eight waves' (m, l, O^T) through LDS.  Partial O^T as float4 quads [d/4][query]: the first half
    // of the columns in this wave's part of Vs0, the second half in its part of Vs1 (each exactly 32 * DV/2 floats).
    half_t* const Vhi = VSINGLE ? Kt : Vs1;            // (one V stage: the K area, as large, takes the second half)
    l = half_sum(l);
    __builtin_amdgcn_s_waitcnt(0x0f70);                 // the look-ahead requests past the end have landed too
    if (h == 0) { st_m[wave][c] = m; st_l[wave][c] = l; }
    if constexpr (NOISE) {
        l2 = half_sum(l2);
        if (h == 0) { st_m2[wave][c] = m2; st_l2[wave][c] = l2; }
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int quad = db * 8 + 2 * r4 + h;             // columns 4 quad .. +3 of this workgroup's share
            float4_t* part = reinterpret_cast<float4_t*>((quad < DV / 8 ? Vs0 : Vhi) + wave * 32 * DV);
            part[(quad % (DV / 8)) * 32 + c] =
                float4_t{oacc[db][r4 * 4], oacc[db][r4 * 4 + 1], oacc[db][r4 * 4 + 2], oacc[db][r4 * 4 + 3]};
        }
    }
    __syncthreads();
    const int q = tid & 31, dg = tid >> 5;                // 16 groups of threads share out the DV/4 quads of a query
    constexpr int NQD = (DV / 4 + 15) / 16;               // quads per thread (with 8 quads, half the groups have none)
    float mstar = st_m[0][q];
#pragma unroll
    for (int w = 1; w < DNW; ++w) mstar = fmaxf(mstar, st_m[w][q]);
    float L = 0.f;
    float4_t acc[NQD];
    {
        float wgt[DNW];
#pragma unroll
        for (int w = 0; w < DNW; ++w) {                   // idle waves: m = -inf, weight 0
            wgt[w] = mstar == -INFINITY ? 0.f : fast_exp2(st_m[w][q] - mstar);
            L += st_l[w][q] * wgt[w];
        }
#pragma unroll
        for (int qi = 0; qi < NQD; ++qi) {
            const int quad = min(dg + 16 * qi, DV / 4 - 1);   // d = 4*quad .. +3 (a group without a quad re-reads the last)
            const half_t* base = quad < DV / 8 ? Vs0 : Vhi;
            const int ql = quad % (DV / 8);
            acc[qi] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < DNW; ++w) acc[qi] += reinterpret_cast<const float4_t*>(base + w * 32 * DV)[ql * 32 + q] * wgt[w];
        }
    }
    float ms2 = -INFINITY, L2 = 0.f;
    if constexpr (NOISE) {
#pragma unroll
        for (int w = 0; w < DNW; ++w) ms2 = fmaxf(ms2, st_m2[w][q]);
#pragma unroll
        for (int w = 0; w < DNW; ++w) L2 += ms2 == -INFINITY ? 0.f : st_l2[w][q] * fast_exp2(st_m2[w][q] - ms2);
    }
    const int bh = b * a.Hq + head;
    if (DS == 1 && a.n_split > 1) {
        // ---- keys split over workgroups: publish (m, l, unnormalised O) of this share; the workgroup that arrives
        // last at the head's counter merges all shares.  Workspace: [arrival counters, 256-byte aligned][bh][split]
        // {O as quads [D/4][32 queries][4], (m, l, m2, l2) [32]} floats.  The shares travel as device-scope atomic stores and loads, which
        // go to the memory all L2 slices agree on (a fence that makes ordinary stores visible writes back and
        // invalidates a whole L2, and with one per wave that took several times the kernel's own time); the arrival
        // is a release/acquire increment by ONE thread, tied to the other threads by the workgroup barriers.
        constexpr int PART = 32 * (D + 4);
        const int n_bh = a.B * a.Hq;
        unsigned* counters = reinterpret_cast<unsigned*>(a.ws);
        float* parts = a.ws + ((n_bh + 63) / 64) * 64;
        float* mine = parts + ((int64_t)bh * a.n_split + split) * PART;
        auto publish = [](float* p, float4_t v) __attribute__((always_inline)) {
            const ulong2_t u = __builtin_bit_cast(ulong2_t, v);
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), u[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(p) + 1, u[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        auto collect = [](const float* p) __attribute__((always_inline)) {
            ulong2_t u;
            u[0] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            u[1] = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return __builtin_bit_cast(float4_t, u);
        };
#pragma unroll
        for (int qi = 0; qi < NQD; ++qi) publish(mine + ((dg + 16 * qi) * 32 + q) * 4, acc[qi]);
        if (dg == 0) publish(mine + 32 * D + 4 * q, float4_t{mstar, L, ms2, L2});
        __syncthreads();                                   // every wave's stores have been acknowledged
        __shared__ unsigned arrival;
        // (release/acquire at device scope makes the hand-over of the shares hold by the memory model alone -- the other
        // threads' stores are ordered before it by the workgroup barrier; it costs one L2 write-back and one invalidate
        // per WORKGROUP, about 1.5 us per launch)
        if (tid == 0) arrival = __hip_atomic_fetch_add(&counters[bh], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (arrival != (unsigned)(a.n_split - 1)) return;
        const float* head_parts = parts + (int64_t)bh * a.n_split * PART;
        // shares are fetched eight at a time (all requests of a batch in flight together) and folded in with a
        // running maximum, in share order: the result does not depend on which workgroup does the merge
        mstar = -INFINITY; ms2 = -INFINITY; L = 0.f; L2 = 0.f;
#pragma unroll
        for (int qi = 0; qi < NQD; ++qi) acc[qi] = float4_t{0.f, 0.f, 0.f, 0.f};
        constexpr int BATCH = 8;
        for (int s0 = 0; s0 < a.n_split; s0 += BATCH) {
            float4_t st[BATCH], d[BATCH][NQD];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const float* ps = head_parts + min(s0 + u, a.n_split - 1) * PART;
                st[u] = collect(ps + 32 * D + 4 * q);
#pragma unroll
                for (int qi = 0; qi < NQD; ++qi) d[u][qi] = collect(ps + ((dg + 16 * qi) * 32 + q) * 4);
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                if (s0 + u >= a.n_split) break;
                const float mnew = fmaxf(mstar, st[u][0]);
                if (mnew > -INFINITY) {                        // -inf: a share that saw no key of this query
                    const float wa = fast_exp2(mstar - mnew), wb = fast_exp2(st[u][0] - mnew);
                    L = L * wa + st[u][1] * wb;
#pragma unroll
                    for (int qi = 0; qi < NQD; ++qi) acc[qi] = acc[qi] * wa + d[u][qi] * wb;
                    mstar = mnew;
                }
                if constexpr (NOISE) {
                    const float m2new = fmaxf(ms2, st[u][2]);
                    if (m2new > -INFINITY) {
                        L2 = L2 * fast_exp2(ms2 - m2new) + st[u][3] * fast_exp2(st[u][2] - m2new);
                        ms2 = m2new;
                    }
                }
            }
        }
        if (tid == 0) __hip_atomic_store(&counters[bh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);                   // left as found: the next launch on the stream starts from zero
    }
    {
        const float inv = 1.0f / L;
        half_t* orow = a.o + b * a.ob + head * a.oh + (int64_t)q * a.os + dsl * DV;
        if (q < a.Sq) {
#pragma unroll
            for (int qi = 0; qi < NQD; ++qi) {
                const half4_t ov = {(half_t)(acc[qi][0] * inv), (half_t)(acc[qi][1] * inv), (half_t)(acc[qi][2] * inv), (half_t)(acc[qi][3] * inv)};
                if (dg + 16 * qi < DV / 4) *reinterpret_cast<half4_t*>(orow + 4 * (dg + 16 * qi)) = ov;
            }
        }
        // (every column share holds the same row normalisers: the first one writes them)
        if (dg == 0 && dsl == 0 && q < a.Sq && a.lse) a.lse[(int64_t)bh * a.Sq + q] = (mstar + fast_log2(L)) * kLn2;
        if constexpr (NOISE) {
            if (dg == 1 && dsl == 0 && q < a.Sq) a.lse_pert[(int64_t)bh * a.Sq + q] = (ms2 + fast_log2(L2)) * kLn2;
        }
    }
    // ---- column statistics (KeyFormer key scores, RoCo sums): a second sweep over this head's keys now that the
    // row normalisers are final.  The score block is formed the other way round, S[query][key] -- the same two
    // register operands with their roles swapped -- so that a lane owns one KEY and holds 16 of the 32 queries: the
    // sum over queries is in-lane plus one exchange with lane^32, and a block's 32 sums are one 128-byte store.
    // (Not with the keys split over workgroups -- the statistics need the normalisers of the whole head; the column
    // shares of a head all have them, and take every DS-th round of blocks of the sweep each.)
    if (a.col_sum || a.col_sumsq || a.probs) {
        __syncthreads();                                   // every thread has read the merge arrays
        if (dg == 0) st_l[0][q] = NOISE ? ms2 + fast_log2(L2) : mstar + fast_log2(L);     // log2 domain
        __syncthreads();
        float lq[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) lq[r] = st_l[0][8 * (r / 4) + 4 * h + (r % 4)];
        const float cs = NOISE ? a.c2 : a.c1;
        // noise of the lane's key for its 16 queries: 16 dwords from 16 rows, consecutive keys in consecutive lanes
        float gs0[NOISE ? 16 : 1], gs1[NOISE ? 16 : 1];
        auto fetch_noise_col = [&](int blk, float (&g)[NOISE ? 16 : 1]) __attribute__((always_inline)) {
            if constexpr (NOISE) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qr = 8 * (r / 4) + 4 * h + (r % 4);
                    if constexpr (N16)
                        g[r] = (float)__builtin_bit_cast(half_t, __builtin_amdgcn_raw_buffer_load_b16(
                            nrs, (int)((qr * a.ns + c) * 2), blk * 64, 0));
                    else
                        g[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                            nrs, (int)((qr * a.ns + c) * 4), blk * 128, 0));
                }
            }
        };
        // (one block ahead is enough: with one workgroup per head the sweep runs at what a single CU can pull from
        // L2, about 55 GB/s; requesting two blocks ahead measured the same)
        auto sweep = [&](int it, half8_t (&kc)[NS], half8_t (&kn)[NS], float (&gc)[NOISE ? 16 : 1], float (&gn)[NOISE ? 16 : 1])
                         __attribute__((always_inline)) {
            const int blk = blk0 + dsl * DNW + wave + it * DNW * DS, key = blk * 32 + c;
            fetch_k(blk + DNW * DS, kn);
            fetch_noise_col(blk + DNW * DS, gn);
            float16_t s;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0.f;
            k_operands(kc);
#pragma unroll
            for (int ks = 0; ks < NS; ++ks) s = mfma32(qB[ks], kc[ks], s);
            float x = 0.f, y = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qr = 8 * (r / 4) + 4 * h + (r % 4);
                float t = __builtin_fmaf(s[r], cs, -lq[r]);
                if constexpr (NOISE) t = __builtin_fmaf(gc[r], a.c3, t);
                const bool ok = key < a.Skv && qr < a.Sq && (!a.causal || key <= qr + off);
                const float p = ok ? fast_exp2(t) : 0.f;
                // (32 consecutive keys of one query row per store instruction: whole 128-byte lines)
                if (a.probs && key < a.Skv && qr < a.Sq) a.probs[((int64_t)bh * a.Sq + qr) * a.Skv + key] = p;
                x += p;
                y = __builtin_fmaf(p, p, y);
            }
            x = half_sum(x); y = half_sum(y);
            if (h == 0 && key < a.Skv) {
                const int64_t at = (int64_t)bh * a.Skv + key;
                if (a.io16) {       // (the fp32 value rounded once, as a copy into the caller's fp16 tensor would)
                    if (a.col_sum) reinterpret_cast<half_t*>(a.col_sum)[at] = (half_t)x;
                    if (a.col_sumsq) reinterpret_cast<half_t*>(a.col_sumsq)[at] = (half_t)y;
                } else {
                    if (a.col_sum) a.col_sum[at] = x;
                    if (a.col_sumsq) a.col_sumsq[at] = y;
                }
            }
        };
        const int first = dsl * DNW + wave;
        const int nsweep = nblk > first ? (nblk - first + DNW * DS - 1) / (DNW * DS) : 0;
        fetch_k(blk0 + first, ka0);
        fetch_noise_col(blk0 + first, gs0);
        for (int it = 0; it < nsweep; it += 2) {
            sweep(it, ka0, ka1, gs0, gs1);
            if (it + 1 < nsweep) sweep(it + 1, ka1, ka0, gs1, gs0);
        }
    }
#endif
}

// Keys are split over workgroups when a head has enough of them to repay the merge (publishing, arriving and collecting
// cost 4 - 5 us) against the unsplit form, whose column shares (up to four workgroups per head) already use half the chip
// at 32 heads.  Measured with 16 queries per head, unsplit / split, us: 32 heads of 128: 2064 keys 13.9 / 22.2, 4112 keys
// 21.5 / 27.1, 8208 keys 36.7 / 35.8, 16400 keys 69 / 57, 65552 keys 406 / 198; 8 heads of 128: 4112 keys 20.0 / 18.1, 8208
// keys 35 / 22, 65552 keys 232 / 59; 71 heads of 64: 4112 keys 14.1 / 14.5, 8208 keys 23.9 / 18.9.  Hence: from 4096 keys
// with at most 16 heads, from 8192 with more, never with 128 heads or more.  The caller provides the workspace for the
// partial results.
static int decode_splits(int batch, int n_q_heads, int seq_kv, int head_dim) {
    const int n_bh = batch * n_q_heads, nblk = (seq_kv + 31) / 32;
    (void)head_dim;
    if (n_bh >= 128 || seq_kv < (n_bh <= 16 ? 4096 : 8192)) return 1;
    const int ns = max(1, min(min(16, 256 / n_bh), nblk / 4));
    const int bps = (nblk + ns - 1) / ns;                 // blocks per share, as the kernel computes it
    return (nblk + bps - 1) / bps;                        // no empty share: the last one starts inside the keys
}

int64_t attn_decode_workspace_bytes(int batch, int n_q_heads, int seq_q, int seq_kv, int head_dim) {
    if (seq_q > 32) return 0;
    const int ns = decode_splits(batch, n_q_heads, seq_kv, head_dim);
    if (ns <= 1) return 0;
    const int64_t n_bh = (int64_t)batch * n_q_heads;
    return ((n_bh + 63) / 64) * 256 + n_bh * ns * 32 * (head_dim + 4) * 4;
}

static int decode_col_shares(int64_t n_bh, int seq_kv, int head_dim) {
    int ds = 1;
    if (seq_kv >= 256)
        while (ds < 4 && head_dim / (ds * 2) >= 32 && n_bh * ds * 2 <= 256) ds *= 2;
    return ds;
}

// Name of the instantiation launched for a problem without a workspace (a measurement aid: what a kernel trace shows).
const char* attn_decode_kernel_name(int batch, int n_q_heads, int seq_kv, int head_dim, bool noise) {
    const int ds = decode_col_shares((int64_t)batch * n_q_heads, seq_kv, head_dim);
    if (head_dim == 128) {
        if (ds == 4) return noise ? "trn::attn_decode_kernel<128, 4, 1>" : "trn::attn_decode_kernel<128, 4, 0>";
        if (ds == 2) return noise ? "trn::attn_decode_kernel<128, 2, 1>" : "trn::attn_decode_kernel<128, 2, 0>";
        return noise ? "trn::attn_decode_kernel<128, 1, 1>" : "trn::attn_decode_kernel<128, 1, 0>";
    }
    if (ds == 2) return noise ? "trn::attn_decode_kernel<64, 2, 1>" : "trn::attn_decode_kernel<64, 2, 0>";
    return noise ? "trn::attn_decode_kernel<64, 1, 1>" : "trn::attn_decode_kernel<64, 1, 0>";
}

hipError_t launch_attn_decode(AttnArgs a, int head_dim, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
    a.n_split = 1; a.ws = nullptr;
    const int64_t need = attn_decode_workspace_bytes(a.B, a.Hq, a.Sq, a.Skv, head_dim);
    if (workspace && need > 0 && workspace_bytes >= need && !a.col_sum && !a.col_sumsq && !a.probs) {
        a.n_split = decode_splits(a.B, a.Hq, a.Skv, head_dim);
        a.ws = static_cast<float*>(workspace);
    }
    // Without a key split: share V's columns out over workgroups while that still leaves every workgroup 32 columns
    // and the grid within one workgroup per CU (32 heads of 128: 4 shares; 71 heads of 64: 2).  Short caches are left
    // alone: below some 8 blocks per wave-round the fixed part of a launch is all there is.
    const int64_t n_bh = (int64_t)a.B * a.Hq;
    const int ds = a.n_split == 1 ? decode_col_shares(n_bh, a.Skv, head_dim) : 1;
    const int64_t grid = ds > 1 ? ((n_bh + 7) / 8) * 8 * ds : n_bh * a.n_split;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 g((unsigned)grid), t(DNW * 64);
#define TRN_DEC(D_, DS_, N_) hipLaunchKernelGGL((attn_decode_kernel<D_, DS_, N_>), g, t, 0, stream, a)
#define TRN_DEC_NZ(D_, DS_) do { if (!a.noise) TRN_DEC(D_, DS_, 0); else if (a.io16) TRN_DEC(D_, DS_, 2); else TRN_DEC(D_, DS_, 1); } while (0)
    if (head_dim == 128) { if (ds == 4) TRN_DEC_NZ(128, 4); else if (ds == 2) TRN_DEC_NZ(128, 2); else TRN_DEC_NZ(128, 1); }
    else { if (ds == 2) TRN_DEC_NZ(64, 2); else TRN_DEC_NZ(64, 1); }
#undef TRN_DEC_NZ
#undef TRN_DEC
    return hipGetLastError();
}

}  // namespace trn

// ---- the entry point that allocates nothing ------------------------------------------------------------------------
// The split-key path needs device memory beyond its inputs and outputs (arrival counters and the shares' partial
// results).  For callers that cannot allocate, that memory is a file-scope device array: every GPU the library runs
// on holds its own copy of it, at its own address, until the process ends.  On the host the array's NAME is only a
// handle for hipGetSymbolAddress; the address that kernels, fills and copies take is the one that call returns for
// the device that is current, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[TRN_ATTN_NOALLOC_SCRATCH_BYTES];

namespace trn {

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];      // device address of `scratch` on each device, null until looked up

// Device address of the scratch array on the current device (looked up on first use; nothing is allocated: the
// array is part of the code object).  Returns nullptr if the runtime refuses.
void* attn_static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

// Zeroes n dwords (a kernel rather than a memset node, so that the call can be recorded into a graph).
__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace trn

extern "C" int trn_attn_fwd_noalloc_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                        float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                        void* stream) {
    using namespace trn;
    if (!d) return TRN_E_NULL;
    const int64_t need = trn_attn_workspace_bytes(d);
    if (need == 0)      // a shape whose kernels use no scratch memory (or an invalid one: reported by the checks below)
        return attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, nullptr, 0, nullptr, nullptr, stream);
    if (need > (int64_t)TRN_ATTN_NOALLOC_SCRATCH_BYTES) return TRN_E_SCRATCH;
    void* ws = attn_static_scratch();
    if (!ws) return TRN_E_LAUNCH;
    // The array keeps whatever the last call on this device left.  The shares are rewritten by every launch before
    // they are read; the arrival counters must start at zero, so they are cleared here (the kernel also leaves them
    // at zero, but a launch that failed half way would not have).
    const int n_counters = (int)(((int64_t)d->batch * d->n_q_heads + 63) / 64) * 64;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((n_counters + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       static_cast<unsigned*>(ws), n_counters);
    if (hipGetLastError() != hipSuccess) return TRN_E_LAUNCH;
    return attn_forward(d, q, k, v, o, lse, gamma_q, noise, lse_pert, ws, TRN_ATTN_NOALLOC_SCRATCH_BYTES, nullptr, nullptr, stream);
}
