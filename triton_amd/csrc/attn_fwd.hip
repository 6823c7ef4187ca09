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
// Workgroup: 256 threads = 4 waves, 128 queries (32 per wave); K/V tiles of BN keys go straight from global
// memory into double-buffered LDS (buffer_load ... lds, no register staging), row-major with an XOR chunk
// swizzle; the V^T A-operand is fetched with the gfx950 transposing LDS read ds_read_b64_tr_b16, so V needs
// no transposition in memory or on the way in.
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


// XOR swizzle of the 16-byte chunk index within a tile row, as a function of the row.  Tiles are stored
// UNPADDED (direct global->LDS loads write 1 KB contiguous per wave instruction), so bank spreading comes from
// the swizzle: it is a bit permutation of the row's low bits chosen so that (a) 16 consecutive rows read at one
// logical chunk (the K operand: one 16-byte read per lane, lane = row) and (b) 4 consecutive rows read over 4
// consecutive chunks (one phase of the transposing V read) both touch every LDS bank exactly once.
template <int D> __device__ __forceinline__ int swz(int r) {
    if constexpr (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);            // 16 chunks per 256-byte row
    else return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);                        // 8 chunks per 128-byte row
}

// One wave's share of a K tile and a V tile: NI wave-wide 1 KB loads each, global -> LDS without passing
// through registers.  Lane i's 16 bytes land at dst + 1024*n + 16*i; which global chunk it fetches (kvo/vvo)
// decides the swizzle.  soffset = tile offset in bytes (wave-uniform).
#if defined(__HIP_DEVICE_COMPILE__)
template <int NI>
__device__ __forceinline__ void fetch_tile(__amdgpu_buffer_rsrc_t krs, __amdgpu_buffer_rsrc_t vrs, half_t* kdst,
                                           half_t* vdst, const int (&kvo)[NI], const int (&vvo)[NI], int ksoff,
                                           int vsoff) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(krs, (__attribute__((address_space(3))) void*)(kdst + i * 512), 16,
                                                 kvo[i], ksoff, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(vrs, (__attribute__((address_space(3))) void*)(vdst + i * 512), 16,
                                                 vvo[i], vsoff, 0, 0);
    }
}
#endif

template <int D, int BN, bool NOISE>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer-descriptor types and LDS-load builtins exist in the device pass only;
                                      // the host pass needs just the launch stub
    constexpr int NKS = D / 16;  // MFMA k-steps over head_dim
    constexpr int NKB = BN / 32; // 32-key blocks per tile
    constexpr int NDB = D / 32;  // 32-wide blocks of head_dim in O^T
    constexpr int CPR = D / 8;   // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;            // tile rows covered by one wave-wide 1 KB load
    constexpr int NI = BN / (RPI * 4);       // such loads per wave per tile (K and V each)
    __shared__ __attribute__((aligned(1024))) half_t Ks[2][BN * D];   // double-buffered: tile j+1 lands while j is used
    __shared__ __attribute__((aligned(1024))) half_t Vs[2][BN * D];

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
    const int qrow = q0 + wave * 32 + c;                // this lane's query
    const int qrow_ld = qrow < a.Sq ? qrow : a.Sq - 1;  // clamp loads; stores are predicated
    const int wave_last_q = min(q0 + wave * 32 + 31, a.Sq - 1);

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

    // ---- LDS read offsets (halfs), lane constants.  K operand: row kb*32+c, logical chunk 2ks+h.
    int koff[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) koff[ks] = c * D + (((2 * ks + h) ^ swz<D>(c)) << 3);
    // V^T operand through the transposing read: in each 16-lane group lanes 4r..4r+3 supply tile row r
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
    float m2 = -INFINITY, l2 = 0.f;    // same for the perturbed scores

    int ntiles = (a.Skv + BN - 1) / BN;
    if (a.causal) ntiles = min(ntiles, (min(q0 + BM - 1, a.Sq - 1) + off) / BN + 1);

    const float* nrow = NOISE ? a.noise + b * a.nb + head * a.nh + (int64_t)qrow_ld * a.ns : nullptr;

    // ---- staging: direct global -> LDS loads, one tile ahead.  Buffer descriptors give zero fill for
    // keys past the end (an all-zero V row times P = 0 contributes nothing; garbage could be NaN).
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.k + b * a.kb + kvh * a.kh), 0, (int)(((int64_t)(a.Skv - 1) * a.ks + D) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.v + b * a.vb + kvh * a.vh), 0, (int)(((int64_t)(a.Skv - 1) * a.vs + D) * 2), 0x00020000);
    int kvo[NI], vvo[NI];       // per-lane byte offsets of this lane's 16-byte chunk within a tile
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int row = (wave * NI + i) * RPI + lane / CPR;
        const int chunk = (lane % CPR) ^ swz<D>(row);        // LDS slot lane%CPR of that row holds this logical chunk
        kvo[i] = (int)(row * a.ks * 2) + chunk * 16;
        vvo[i] = (int)(row * a.vs * 2) + chunk * 16;
    }
    const int ktile_bytes = (int)(BN * a.ks * 2), vtile_bytes = (int)(BN * a.vs * 2);
    // (a __device__ function, not a lambda: with the LDS-load builtin inside a lambda in this kernel template
    // the host pass silently drops the kernel's launch stub)
#define TRN_FETCH(jt_, buf_) fetch_tile<NI>(krs, vrs, &Ks[buf_][wave * NI * 512], &Vs[buf_][wave * NI * 512], kvo, vvo, \
                                           (jt_) * ktile_bytes, (jt_) * vtile_bytes)
    TRN_FETCH(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0f70);     // vmcnt(0): this wave's loads have landed in LDS
    __syncthreads();

    for (int jt = 0; jt < ntiles; ++jt) {
        const int kv0 = jt * BN, cur = jt & 1;
        if (jt + 1 < ntiles) TRN_FETCH(jt + 1, cur ^ 1);   // lands during this tile's MFMAs; last readers of that
                                                       // buffer passed the barrier that ended the previous tile

        // whole tile masked for this wave (wave-uniform)?  It still stages and meets the barrier.
        if (!(a.causal && kv0 > wave_last_q + off)) {
            const half_t* Kc = Ks[cur];
            const half_t* Vc = Vs[cur];
            // ---- S^T = K Q^T ----
            float16_t sacc[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
                const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    half8_t ka = *reinterpret_cast<const half8_t*>(&Kc[kb * 32 * D + koff[ks]]);
                    sacc[kb] = mfma32(ka, qB[ks], ks == 0 ? zero : sacc[kb]);
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

            // ---- online softmax (log2 domain) against a LAZY reference max ----
            // m is only raised when some row's true running max exceeds it by more than 2^8: probabilities
            // are then at most 256 (exact in fp16's range, fp32 sums), O and l stay relative to the same m so
            // the final O/l and m + log2(l) are unchanged, and the 16*NDB-multiply rescale of O^T -- a large
            // share of the VALU work -- runs on the first tile or two only instead of on most tiles.
            float smax = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) smax = fmaxf(smax, sacc[kb][r]);
            smax = half_max(smax) * a.c1;
            if (__builtin_amdgcn_ballot_w64(smax > m + 8.0f) != 0) {      // wave-uniform
                const float mnew = fmaxf(m, smax);
                const float alpha = fast_exp2(m - mnew);
                l *= alpha;
#pragma unroll
                for (int i = 0; i < NDB; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
                m = mnew;
            }

            // ---- P^T (fp16) straight into B-operands, O^T += V^T P^T ----
            // The row sum is taken over the fp16-rounded P (v_dot2_f32_f16 against ones, fp32 accumulate),
            // i.e. over exactly the values that multiply V.
            const half2_t ones = {(half_t)1.f, (half_t)1.f};
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
                for (int sp = 0; sp < 2; ++sp) {
                    half8_t pB;
#pragma unroll
                    for (int t = 0; t < 8; t += 2) {
                        const float p0 = fast_exp2(__builtin_fmaf(sacc[kb][8 * sp + t], a.c1, -m));
                        const float p1 = fast_exp2(__builtin_fmaf(sacc[kb][8 * sp + t + 1], a.c1, -m));
                        const half2_t pp = {(half_t)p0, (half_t)p1};
                        l = __builtin_amdgcn_fdot2(pp, ones, l, false);
                        pB[t] = pp[0]; pB[t + 1] = pp[1];
                    }
#pragma unroll
                    for (int db = 0; db < NDB; ++db) {
                        const half_t* vp = &Vc[(kb * 32 + 16 * sp) * D];
                        half4_t lo = lds_read_tr16(vp + voff_lo[db]);   // keys +0..3 of this lane half, dim db*32+c
                        half4_t hi = lds_read_tr16(vp + voff_hi[db]);   // keys +8..11
                        half8_t va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        oacc[db] = mfma32(va, pB, oacc[db]);
                    }
                }
            }
        }

        __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): this wave's share of the next tile is in LDS
        __syncthreads();                      // next tile visible; this tile's buffer may be overwritten next time
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
        if (h == 0 && a.lse) a.lse[((int64_t)b * a.Hq + head) * a.Sq + qrow] = (m + fast_log2(l)) * kLn2;
    }
    if constexpr (NOISE) {
        const float l2s = half_sum(l2);
        if (qrow < a.Sq && h == 0)
            a.lse_pert[((int64_t)b * a.Hq + head) * a.Sq + qrow] = (m2 + fast_log2(l2s)) * kLn2;
    }
#endif
}

#undef TRN_FETCH

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
    // K/V tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base
    if (((int64_t)d->seq_kv + 128) * d->k_stride_s * 2 > 0x7fffffffLL || ((int64_t)d->seq_kv + 128) * d->v_stride_s * 2 > 0x7fffffffLL)
        return TRN_E_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (d->head_dim == 128) e = noise ? launch_fwd<128, 64, true>(a, s) : launch_fwd<128, 64, false>(a, s);
    else e = noise ? launch_fwd<64, 64, true>(a, s) : launch_fwd<64, 64, false>(a, s);
    return e == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}
