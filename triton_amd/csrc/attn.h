// Argument block shared by the attention forward kernels.
#pragma once
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

// At most 32 queries per head (decode): one workgroup per head whose eight waves split the keys (attn_decode.hip).
hipError_t launch_attn_decode(const AttnArgs& a, int head_dim, hipStream_t stream);

}  // namespace trn
