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
};

constexpr int CBN = 128;  // keys per workgroup
constexpr int CBM = 64;   // queries per staged tile

template <int D, bool NOISE>
__global__ __launch_bounds__(256, 2) void attn_colstats_kernel(const ColArgs a) {
    constexpr int QP = D + 8;
    constexpr int NKS = D / 16;
    __shared__ __attribute__((aligned(16))) half_t Qs[CBM * QP];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;
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

    float s1[16], s2[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { s1[r] = 0.f; s2[r] = 0.f; }

    const half_t* qbase = a.q + b * a.qb + head * a.qh;
    const float* lrow = a.lse + ((int64_t)b * a.Hq + head) * a.Sq;
    const float* nbase = NOISE ? a.noise + b * a.nb + head * a.nh : nullptr;

    const int first_q = a.causal ? max(0, kv0 - off) : 0;   // earlier queries see none of this tile's keys
    for (int q0 = (first_q / CBM) * CBM; q0 < a.Sq; q0 += CBM) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < (CBM * D / 8) / 256; ++i) {
            const int id = tid + i * 256, row = id / (D / 8), c8 = id % (D / 8);
            const int qr = q0 + row;
            uint4_t val = {0u, 0u, 0u, 0u};
            if (qr < a.Sq) val = *reinterpret_cast<const uint4_t*>(qbase + (int64_t)qr * a.qs + c8 * 8);
            *reinterpret_cast<uint4_t*>(&Qs[row * QP + c8 * 8]) = val;
        }
        __syncthreads();
        // queries of this tile all earlier than this wave's first key: nothing visible (wave-uniform)
        if (a.causal && q0 + CBM - 1 + off < wkey0) continue;

#pragma unroll
        for (int qb = 0; qb < CBM / 32; ++qb) {
            const int qrow = q0 + qb * 32 + c;
            float16_t acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                half8_t qv = *reinterpret_cast<const half8_t*>(&Qs[(qb * 32 + c) * QP + ks * 16 + 8 * h]);
                acc = mfma32(kA[ks], qv, acc);
            }
            const bool qok = qrow < a.Sq;
            const float lse2 = qok ? lrow[qrow] * kLog2e : 0.f;
            const float* nrow = NOISE ? nbase + (int64_t)(qok ? qrow : 0) * a.ns : nullptr;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int key0 = wkey0 + 8 * r4 + 4 * h;
                float4_t gv = {0.f, 0.f, 0.f, 0.f};
                if constexpr (NOISE) {
                    if (qok && key0 < a.Skv && (!a.causal || key0 <= qrow + off)) {
                        if (key0 + 3 < a.Skv) gv = *reinterpret_cast<const float4_t*>(nrow + key0);
                        else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) if (key0 + e < a.Skv) gv[e] = nrow[key0 + e];
                        }
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = key0 + e;
                    const bool ok = qok && key < a.Skv && (!a.causal || key <= qrow + off);
                    float t = __builtin_fmaf(acc[r4 * 4 + e], a.c1, -lse2);
                    if constexpr (NOISE) t = __builtin_fmaf(gv[e], a.c3, t);
                    const float p = ok ? fast_exp2(t) : 0.f;
                    s1[r4 * 4 + e] += p;
                    s2[r4 * 4 + e] += p * p;
                }
            }
        }
    }

    // sum over the 32 queries held by lanes c = 0..31 (same h), then lane c == 0 of each half writes
    const int64_t obase = ((int64_t)b * a.Hq + head) * a.Skv;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        float x = s1[r], y = s2[r];
#pragma unroll
        for (int msk = 1; msk < 32; msk <<= 1) { x += __shfl_xor(x, msk, 64); y += __shfl_xor(y, msk, 64); }
        const int key = wkey0 + 8 * (r / 4) + 4 * h + (r % 4);
        if (c == 0 && key < a.Skv) {
            if (a.out_sum) a.out_sum[obase + key] = x;
            if (a.out_sumsq) a.out_sumsq[obase + key] = y;
        }
    }
}

template <int D, bool NOISE>
static hipError_t launch_col(const ColArgs& a, hipStream_t s) {
    const unsigned grid = (unsigned)a.n_kvtiles * a.B * a.Hq;
    hipLaunchKernelGGL((attn_colstats_kernel<D, NOISE>), dim3(grid), dim3(256), 0, s, a);
    return hipGetLastError();
}

}  // namespace trn

extern "C" int trn_attn_colstats_f16(const trn_attn_desc* d, const void* q, const void* k, const float* lse,
                                     const float* noise, float* out_sum, float* out_sumsq, void* stream) {
    using namespace trn;
    if (!d || !q || !k || !lse) return TRN_E_NULL;
    if (!out_sum && !out_sumsq) return TRN_E_NULL;
    int st = validate_attn(d, false);
    if (st != TRN_OK) return st;
    if (d->q_norm) return TRN_E_UNSUPPORTED;
    if (!aligned16(q) || !aligned16(k)) return TRN_E_ALIGN;
    if (noise) {
        if (!(d->tau > 0.f)) return TRN_E_UNSUPPORTED;
        if (d->noise_stride_s < d->seq_kv) return TRN_E_STRIDE;
        if (!aligned16(noise) || !pitch16(d->noise_stride_s, 4) || !pitch16(d->noise_stride_h, 4) ||
            !pitch16(d->noise_stride_b, 4))
            return TRN_E_ALIGN;
    }
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
    if ((int64_t)a.n_kvtiles * a.B * a.Hq > 0x7fffffffLL) return TRN_E_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (d->head_dim == 128) e = noise ? launch_col<128, true>(a, s) : launch_col<128, false>(a, s);
    else e = noise ? launch_col<64, true>(a, s) : launch_col<64, false>(a, s);
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
