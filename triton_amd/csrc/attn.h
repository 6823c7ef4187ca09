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
    // decode kernel only: keys split over n_split workgroups per head, partial results and arrival counters in ws
    int n_split;
    float* ws;
    // decode kernel only, one workgroup per head: per-key sums (and sums of squares) of the probabilities -- of the
    // perturbed ones when noise is given -- from a second sweep over the keys once the row normalisers are final
    float* col_sum; float* col_sumsq;
    // ... and the probabilities themselves, un-reduced: float [B, Hq, Sq, Skv] contiguous
    float* probs;
    // decode kernel only: noise, col_sum and col_sumsq point at fp16 data (noise pitches in halfs)
    int io16;
};

// Checks, argument block and kernel choice behind every attention entry point of the C ABI.
int attn_forward(const trn_attn_desc* d, const void* q, const void* k, const void* v, void* o, float* lse,
                 const void* gamma_q, const float* noise, float* lse_pert, void* workspace,
                 int64_t workspace_bytes, float* col_sum, float* col_sumsq, void* stream, float* probs = nullptr,
                 bool io16 = false);

// At most 32 queries per head (decode): one workgroup per head whose eight waves split the keys (attn_decode.hip).
hipError_t launch_attn_decode(AttnArgs a, int head_dim, void* workspace, int64_t workspace_bytes, hipStream_t stream);
const char* attn_decode_kernel_name(int batch, int n_q_heads, int seq_kv, int head_dim, bool noise);
// Bytes of workspace with which launch_attn_decode splits the keys of this problem over several workgroups (0: it would not).
int64_t attn_decode_workspace_bytes(int batch, int n_q_heads, int seq_q, int seq_kv, int head_dim);

// Device address, on the current device, of the library's static scratch array (TRN_ATTN_NOALLOC_SCRATCH_BYTES bytes)
// behind trn_attn_fwd_noalloc_f16; looked up once per device.  nullptr if the runtime refuses.
void* attn_static_scratch();

// The forward pass without score perturbation on the 16x16x32 MFMA (attn_fwd16.hip).  Narrow: 4 waves x 32 queries
// per workgroup; Wide: 8 waves x 32 consecutive queries; Paired: 8 waves, two 128-query tiles from opposite ends of
// the sequence (causal problems whose grid is a single round).
enum class Attn16Shape { Narrow, Wide, Paired };
Attn16Shape attn_fwd16_shape(int batch, int n_q_heads, int seq_q, int head_dim, bool causal);
hipError_t launch_attn_fwd16(const AttnArgs& a, int head_dim, Attn16Shape shape, hipStream_t stream);
// Name of the kernel instantiation that launch_attn_fwd16 runs for this shape, as a profiler prints it.
const char* attn_fwd16_kernel_name(int head_dim, Attn16Shape shape);

}  // namespace trn
