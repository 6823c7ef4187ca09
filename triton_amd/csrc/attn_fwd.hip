// Flash attention forward for gfx950: O = softmax(scale * Q K^T [+causal]) V, GQA/MQA, head_dim 64/128.
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
// Workgroup: 256 threads = 4 waves, 128 queries (32 per wave); K/V tiles of BN keys staged through LDS
// (both row-major, padded; the V^T A-operand is fetched with the gfx950 transposing LDS read
// ds_read_b64_tr_b16, so V needs no transposition in memory or on the way in).
// Grid: one workgroup per (query tile, batch, head), heaviest (latest) query tiles first; consecutive
// workgroup ids map to different KV heads so that the query heads sharing a KV head land on the same XCD
// (ids are dealt round-robin to the 8 XCDs) and hit its L2.
#include "common.h"

namespace trn {

struct AttnArgs {
    const half_t* q; const half_t* k; const half_t* v; half_t* o;
    float* lse; const half_t* gamma_q; const float* noise; float* lse_pert;
    int B, Hq, Hkv, Sq, Skv, n_qtiles;
    int64_t qb, qh, qs, kb, kh, ks, vb, vh, vs, ob, oh, os, nb, nh, ns;
    float c1;      // scale * log2(e)                    : plain scores in the log2 domain
    float c2, c3;  // scale*log2(e)/tau, log2(e)/tau     : perturbed scores  z2 = s*c2 + g*c3
    float q_eps;
    int causal, q_norm;
};

constexpr int BM = 128;


template <int D, int BN, bool NOISE>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnArgs a) {
    constexpr int KP = D + 8;    // K tile pitch in halfs: 16 B pad -> conflict-free 16 B row reads
    constexpr int NKS = D / 16;  // MFMA k-steps over head_dim
    constexpr int NKB = BN / 32; // 32-key blocks per tile
    constexpr int NDB = D / 32;  // 32-wide blocks of head_dim in O^T
    __shared__ __attribute__((aligned(16))) half_t Ks[BN * KP];
    __shared__ __attribute__((aligned(16))) half_t Vs[BN * KP];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;

    // ---- which (query tile, batch, head): heavy tiles first, KV heads interleaved across ids
    const int BH = a.B * a.Hq;
    const int qt = a.n_qtiles - 1 - (int)(blockIdx.x / BH);
    const int j = blockIdx.x % BH;
    const int G = a.Hq / a.Hkv, nkv = a.B * a.Hkv;
    const int kvslot = j % nkv, g = j / nkv;
    const int b = kvslot / a.Hkv, kvh = kvslot % a.Hkv, head = kvh * G + g;

    const int off = a.Skv - a.Sq;                       // causal: query i sees keys <= i + off
    const int q0 = qt * BM;
    const int qrow = q0 + wave * 32 + c;                // this lane's query
    const int qrow_ld = qrow < a.Sq ? qrow : a.Sq - 1;  // clamp loads; stores are predicated
    const int wave_last_q = min(q0 + wave * 32 + 31, a.Sq - 1);
    // transposing-read address pattern: lane supplies row (lane%16)/4, 4 columns at 16*((lane%32)/16) + 4*(lane%4)
    const int tr_row = (lane & 15) >> 2, tr_col = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;

    // ---- Q^T B-operands: lane holds Q[qrow][ks*16 + 8h .. +7]
    half8_t qB[NKS];
    {
        const half_t* qp = a.q + b * a.qb + head * a.qh + (int64_t)qrow_ld * a.qs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) qB[ks] = *reinterpret_cast<const half8_t*>(qp + ks * 16);
        if (a.q_norm) {   // fused per-head RMSNorm of the query row (other half of the row is in lane^32)
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e) { float f = (float)qB[ks][e]; ss += f * f; }
            ss = half_sum(ss);
            const float rstd = 1.0f / __builtin_sqrtf(ss / (float)D + a.q_eps);
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
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

    float16_t oacc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;      // running max (log2 domain) and this lane's partial row sum
    float m2 = -INFINITY, l2 = 0.f;    // same for the perturbed scores

    int ntiles = (a.Skv + BN - 1) / BN;
    if (a.causal) ntiles = min(ntiles, (min(q0 + BM - 1, a.Sq - 1) + off) / BN + 1);

    const half_t* kbase = a.k + b * a.kb + kvh * a.kh;
    const half_t* vbase = a.v + b * a.vb + kvh * a.vh;
    const float* nrow = NOISE ? a.noise + b * a.nb + head * a.nh + (int64_t)qrow_ld * a.ns : nullptr;

    for (int jt = 0; jt < ntiles; ++jt) {
        const int kv0 = jt * BN;
        __syncthreads();   // previous tile fully consumed
        // ---- stage K tile (row-major) ----
#pragma unroll
        for (int i = 0; i < (BN * D / 8) / 256; ++i) {
            const int id = tid + i * 256, row = id / (D / 8), c8 = id % (D / 8);
            const int key = kv0 + row;
            uint4_t val = {0u, 0u, 0u, 0u};
            if (key < a.Skv) val = *reinterpret_cast<const uint4_t*>(kbase + (int64_t)key * a.ks + c8 * 8);
            *reinterpret_cast<uint4_t*>(&Ks[row * KP + c8 * 8]) = val;
        }
        // ---- stage V tile (row-major) ----
#pragma unroll
        for (int i = 0; i < (BN * D / 8) / 256; ++i) {
            const int id = tid + i * 256, row = id / (D / 8), c8 = id % (D / 8);
            const int key = kv0 + row;
            uint4_t val = {0u, 0u, 0u, 0u};      // keys past the end must be 0, not garbage: 0 * NaN = NaN
            if (key < a.Skv) val = *reinterpret_cast<const uint4_t*>(vbase + (int64_t)key * a.vs + c8 * 8);
            *reinterpret_cast<uint4_t*>(&Vs[row * KP + c8 * 8]) = val;
        }
        __syncthreads();

        if (a.causal && kv0 > wave_last_q + off) continue;   // whole tile masked for this wave (wave-uniform)

        // ---- S^T = K Q^T ----
        float16_t sacc[NKB];
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                half8_t ka = *reinterpret_cast<const half8_t*>(&Ks[(kb * 32 + c) * KP + ks * 16 + 8 * h]);
                sacc[kb] = mfma32(ka, qB[ks], sacc[kb]);
            }
        }

        // ---- perturbed-score row normaliser (KeyFormer): z2 = s*c2 + g*c3, online (m2, l2) ----
        if constexpr (NOISE) {
            float zmax = m2;
            float16_t z[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int key0 = kv0 + kb * 32 + 8 * r4 + 4 * h;
                    float4_t gv = {0.f, 0.f, 0.f, 0.f};
                    const bool any_visible = key0 < a.Skv && (!a.causal || key0 <= qrow + off);
                    if (any_visible) {
                        if (key0 + 3 < a.Skv) gv = *reinterpret_cast<const float4_t*>(nrow + key0);
                        else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) if (key0 + e < a.Skv) gv[e] = nrow[key0 + e];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int key = key0 + e;
                        const bool ok = key < a.Skv && (!a.causal || key <= qrow + off);
                        float zz = sacc[kb][r4 * 4 + e] * a.c2 + gv[e] * a.c3;
                        zz = ok ? zz : -INFINITY;
                        z[kb][r4 * 4 + e] = zz;
                        zmax = fmaxf(zmax, zz);
                    }
                }
            zmax = half_max(zmax);
            float sum = 0.f;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += fast_exp2(z[kb][r] - zmax);
            l2 = l2 * fast_exp2(m2 - zmax) + sum;
            m2 = zmax;
        }

        // ---- mask (diagonal / ragged tiles only) ----
        const bool need_mask = (kv0 + BN > a.Skv) || (a.causal && kv0 + BN - 1 > q0 + wave * 32 + off);
        if (need_mask) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kv0 + kb * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                    const bool ok = key < a.Skv && (!a.causal || key <= qrow + off);
                    sacc[kb][r] = ok ? sacc[kb][r] : -INFINITY;
                }
        }

        // ---- online softmax (log2 domain) ----
        float smax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) smax = fmaxf(smax, sacc[kb][r]);
        smax = half_max(smax);
        const float mnew = fmaxf(m, smax * a.c1);
        const float alpha = fast_exp2(m - mnew);
        m = mnew;
        l *= alpha;
#pragma unroll
        for (int i = 0; i < NDB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;

        // ---- P^T (fp16) straight into B-operands, O^T += V^T P^T ----
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
            for (int sp = 0; sp < 2; ++sp) {
                half8_t pB;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const float p = fast_exp2(__builtin_fmaf(sacc[kb][8 * sp + t], a.c1, -mnew));
                    l += p;
                    pB[t] = (half_t)p;
                }
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    const half_t* vp = &Vs[(kb * 32 + 16 * sp + 4 * h + tr_row) * KP + db * 32 + tr_col];
                    half4_t lo = lds_read_tr16(vp);            // keys +0..3 of this lane half, dim db*32+c
                    half4_t hi = lds_read_tr16(vp + 8 * KP);   // keys +8..11
                    half8_t va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    oacc[db] = mfma32(va, pB, oacc[db]);
                }
            }
        }
    }

    // ---- epilogue: normalise, store O[qrow][d..d+3], LSEs ----
    l = half_sum(l);
    const float inv = 1.0f / l;
    if (qrow < a.Sq) {
        half_t* op = a.o + b * a.ob + head * a.oh + (int64_t)qrow * a.os;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                half4_t ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) ov[e] = (half_t)(oacc[db][r4 * 4 + e] * inv);
                *reinterpret_cast<half4_t*>(op + db * 32 + 8 * r4 + 4 * h) = ov;
            }
        if (h == 0) {
            const int64_t li = ((int64_t)b * a.Hq + head) * a.Sq + qrow;
            if (a.lse) a.lse[li] = (m + fast_log2(l)) * kLn2;
        }
    }
    if constexpr (NOISE) {
        const float l2s = half_sum(l2);
        if (qrow < a.Sq && h == 0)
            a.lse_pert[((int64_t)b * a.Hq + head) * a.Sq + qrow] = (m2 + fast_log2(l2s)) * kLn2;
    }
}

template <int D, int BN, bool NOISE>
static hipError_t launch_fwd(const AttnArgs& a, hipStream_t s) {
    const unsigned grid = (unsigned)a.n_qtiles * a.B * a.Hq;
    hipLaunchKernelGGL((attn_fwd_kernel<D, BN, NOISE>), dim3(grid), dim3(256), 0, s, a);
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

extern "C" int trn_attn_fwd_f16(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o,
                                float* lse, const void* gamma_q, const float* noise, float* lse_pert,
                                void* stream) {
    using namespace trn;
    if (!d || !q || !k || !v || !o) return TRN_E_NULL;
    if (noise && !lse_pert) return TRN_E_NULL;
    int st = validate_attn(d, true);
    if (st != TRN_OK) return st;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || (gamma_q && !aligned16(gamma_q)))
        return TRN_E_ALIGN;
    if (noise) {
        if (!(d->tau > 0.f)) return TRN_E_UNSUPPORTED;
        if (d->noise_stride_s < d->seq_kv) return TRN_E_STRIDE;
        if (!aligned16(noise) || !pitch16(d->noise_stride_s, 4) || !pitch16(d->noise_stride_h, 4) ||
            !pitch16(d->noise_stride_b, 4))
            return TRN_E_ALIGN;
    }
    AttnArgs a;
    a.q = (const half_t*)q; a.k = (const half_t*)k; a.v = (const half_t*)v; a.o = (half_t*)o;
    a.lse = lse; a.gamma_q = (const half_t*)gamma_q; a.noise = noise; a.lse_pert = lse_pert;
    a.B = d->batch; a.Hq = d->n_q_heads; a.Hkv = d->n_kv_heads; a.Sq = d->seq_q; a.Skv = d->seq_kv;
    a.n_qtiles = (d->seq_q + BM - 1) / BM;
    a.qb = d->q_stride_b; a.qh = d->q_stride_h; a.qs = d->q_stride_s;
    a.kb = d->k_stride_b; a.kh = d->k_stride_h; a.ks = d->k_stride_s;
    a.vb = d->v_stride_b; a.vh = d->v_stride_h; a.vs = d->v_stride_s;
    a.ob = d->o_stride_b; a.oh = d->o_stride_h; a.os = d->o_stride_s;
    a.nb = d->noise_stride_b; a.nh = d->noise_stride_h; a.ns = d->noise_stride_s;
    a.c1 = d->scale * kLog2e;
    const float tau = noise ? d->tau : 1.f;
    a.c2 = d->scale * kLog2e / tau; a.c3 = kLog2e / tau;
    a.q_eps = d->q_norm_eps; a.causal = d->causal ? 1 : 0; a.q_norm = d->q_norm ? 1 : 0;
    if ((int64_t)a.n_qtiles * a.B * a.Hq > 0x7fffffffLL) return TRN_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (d->head_dim == 128) e = noise ? launch_fwd<128, 64, true>(a, s) : launch_fwd<128, 64, false>(a, s);
    else e = noise ? launch_fwd<64, 64, true>(a, s) : launch_fwd<64, 64, false>(a, s);
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
