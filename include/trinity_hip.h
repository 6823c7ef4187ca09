/*
 * trinity_hip.h -- C ABI of libtrinity_hip.so: hand-written gfx950 (MI355X) kernels for the
 * fused operators that the reference's code generator emits at run time.
 *
 * Boundary being replaced.  In the reference a generated Python module exposes
 * `forward(*tensors, **block_sizes)` (TritonGen.py:568-712) whose body launches
 * `kernel_i[grid](ptr, ptr.stride(0), ..., M=..., N=..., D=..., H=..., P=...)` on the
 * caller's current stream (TritonGen.py:590-708).  Each function below is what one such
 * launch becomes: plain device pointers, element strides and sizes in; results written in
 * place into caller-owned buffers; enqueued on the stream handle given; nothing allocated,
 * nothing synchronised, no host read of device memory -- so a call may sit inside a HIP
 * graph capture exactly as the reference's callers capture `forward`
 * (vanilla_llama_benchmark.py:254-285).
 *
 * Conventions
 *   - All tensors are fp16 unless a parameter says float.  Innermost (feature) stride is 1.
 *   - Strides are in ELEMENTS.  Base pointers and row pitches must be 16-byte aligned
 *     (128-bit loads); otherwise TRN_E_ALIGN.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *   - Every function returns TRN_OK or a negative trn_status; it never throws or aborts.
 *   - Query head h reads KV head h / (n_q_heads / n_kv_heads)  (GQA / MQA).
 *   - Causal with seq_q < seq_kv: query i sees keys j <= i + (seq_kv - seq_q)  (cached prefix).
 */
#ifndef TRINITY_HIP_H
#define TRINITY_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum trn_status {
    TRN_OK            =  0,
    TRN_E_NULL        = -1,  /* a required pointer is NULL                              */
    TRN_E_SHAPE       = -2,  /* a size is <= 0, not a supported multiple, or inconsistent */
    TRN_E_STRIDE      = -3,  /* a stride is too small for the shape                       */
    TRN_E_ALIGN       = -4,  /* pointer or pitch not 16-byte aligned                      */
    TRN_E_UNSUPPORTED = -5,  /* e.g. head_dim not in {64,128}                             */
    TRN_E_LAUNCH      = -6,  /* the HIP runtime refused the launch                        */
    TRN_E_ARCH        = -7,  /* current device is not gfx950                              */
    TRN_E_SCRATCH     = -8   /* the problem needs more scratch memory than the library's static buffer holds */
} trn_status;

/* Library version (major*10000 + minor*100 + patch). */
int trn_version(void);

/* Static string naming a trn_status value ("TRN_E_SHAPE"...). */
const char* trn_status_name(int status);

/* 0 if the current HIP device is a gfx950, TRN_E_ARCH otherwise.  Also looks up, for this device, the
 * address of the static scratch array behind trn_attn_fwd_noalloc_f16.  Not capture-safe (queries
 * device properties); call once per device at load time. */
int trn_check_device(void);

/*
 * RMSNorm rows:  y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * gamma[:]
 * Replaces the arithmetic of ref_attn.py:348-350 (eps + weight form) and ref_rms.py:102-103
 * (gamma == NULL, eps == 0).  fp32 mean-square; x is read once and y written once.
 *
 * Rows are addressed in two levels so the same kernel serves per-head normalisation of a
 * [heads, seq, head_dim] tensor from row `row_start` on (ref_rms.py:217-222: only the
 * newly appended keys are normalised):
 *     row r -> outer = r / inner_rows, inner = r % inner_rows
 *     x + outer*x_outer_stride + (row_start + inner)*ldx ;  y likewise.
 * A plain [rows, cols] matrix is outer_rows = 1, inner_rows = rows, row_start = 0.
 * cols must be a multiple of 8 and <= 16384.  y may be x itself (in place); gamma must not overlap y.
 */
int trn_rmsnorm_f16(const void* x, const void* gamma /* nullable */, void* y,
                    int64_t outer_rows, int64_t inner_rows, int64_t cols,
                    int64_t x_outer_stride, int64_t ldx,
                    int64_t y_outer_stride, int64_t ldy,
                    int64_t row_start, float eps, void* stream);

/* Shape / layout of one attention problem.  q,o: [batch, n_q_heads, seq_q, head_dim];
 * k,v: [batch, n_kv_heads, seq_kv, head_dim]; any of them may be a strided view
 * (e.g. token-major [batch, seq, heads*head_dim] has *_stride_h = head_dim). */
typedef struct trn_attn_desc {
    int32_t batch, n_q_heads, n_kv_heads, seq_q, seq_kv, head_dim;
    int64_t q_stride_b, q_stride_h, q_stride_s;
    int64_t k_stride_b, k_stride_h, k_stride_s;
    int64_t v_stride_b, v_stride_h, v_stride_s;
    int64_t o_stride_b, o_stride_h, o_stride_s;
    float   scale;        /* multiplies Q K^T; the reference classes use 1 (ref_rms.py:77) */
    int32_t causal;       /* 0: every query sees every key (ref_rms.py:78); 1: causal      */
    /* Fused per-head RMSNorm of Q over head_dim before Q K^T (ref_rms.py:217-219). */
    int32_t q_norm;       /* 0 off, 1 on                                                   */
    float   q_norm_eps;
    /* KeyFormer perturbation (ref_rms.py:172): z = (scale*QK^T + noise) / tau.            */
    int64_t noise_stride_b, noise_stride_h, noise_stride_s;   /* noise [b, hq, seq_q, seq_kv] float; base and all
                                                                 three pitches multiples of 16 bytes (seq_kv itself
                                                                 may be anything: pad the rows)                   */
    float   tau;
} trn_attn_desc;

/*
 * O = softmax(scale * Q K^T [+ causal mask]) V, fp32 softmax and accumulation, one pass over
 * K/V with online softmax (no S x S intermediate).  Replaces the kernels generated for
 * ref_rms.py:77-80 (Vanila), :225-228 (QKNorm, with q_norm=1 and K normalised beforehand by
 * trn_rmsnorm_f16), and the attention half of :121-124 (PreNorm), :171-176 (KeyFormer),
 * :272-277 (RoCo).
 *
 *   lse        nullable float [batch, n_q_heads, seq_q] (contiguous): natural-log row
 *              normaliser log sum_j exp(s_ij), needed by trn_attn_colstats_f16.
 *   gamma_q    nullable fp16 [head_dim]: weight of the fused Q norm (used when q_norm=1).
 *   noise      nullable float: when given, the kernel also reduces the row normaliser of the
 *              perturbed scores z into lse_pert (same shape as lse; required then).
 */
int trn_attn_fwd_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                     void* o, float* lse, const void* gamma_q,
                     const float* noise, float* lse_pert, void* stream);

/*
 * trn_attn_fwd_f16 with a caller-provided workspace.  In the reference every cross-kernel intermediate is a
 * caller-allocated tensor passed to `forward` (C, C_exp, C_sum ... in vanilla_llama_benchmark.py:42-77, zero-filled
 * by the driver, :237-240); this is that convention for the one intermediate these kernels have.  For decode shapes
 * (seq_q <= 32) with fewer than 128 heads on a long cache (4096 keys or more with at most 16 heads, 8192 or more
 * otherwise) the keys are then split over several workgroups per head, whose partial results and
 * arrival counters live in the workspace; for every other shape, or with workspace == NULL or too small, the call is
 * exactly trn_attn_fwd_f16.
 *   workspace        device memory, 256-byte aligned, trn_attn_workspace_bytes(desc) bytes, zero-filled ONCE before
 *                    its first use (the kernel returns its counters to zero).  One call at a time may use it.
 * trn_attn_workspace_bytes returns 0 when the shape would not use a workspace.
 */
int64_t trn_attn_workspace_bytes(const trn_attn_desc* desc);
int trn_attn_fwd_ws_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                        void* o, float* lse, const void* gamma_q,
                        const float* noise, float* lse_pert,
                        void* workspace, int64_t workspace_bytes, void* stream);

/*
 * trn_attn_fwd_ws_f16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): it has no counterpart in the reference.  The workspace is a static device
 * array inside the library, TRN_ATTN_NOALLOC_SCRATCH_BYTES per GPU, held from load until the process ends; the call
 * itself allocates and frees nothing.  A problem whose workspace (trn_attn_workspace_bytes) would be larger is
 * rejected with TRN_E_SCRATCH; one that needs none runs as trn_attn_fwd_f16.  (With the present split rule -- at most
 * 256 shares over all heads, 32 x (head_dim + 4) floats each, head_dim <= 128 -- no workspace exceeds 4.4 MB, so the
 * rejection cannot occur today; it guards a future rule, and a host-side test sweeps trn_attn_workspace_bytes over the
 * supported shapes against the array's size.)  The arrival counters are cleared by a
 * small kernel on `stream` before the attention kernel, so a call does not depend on what the previous one left.
 * All calls on one GPU share the one array: calls that overlap on a GPU (two streams, two threads) race; serialise
 * them, or give overlapping callers their own workspace through trn_attn_fwd_ws_f16.  Call trn_check_device once
 * per device first if the call is to be captured into a graph (the first call on a device otherwise looks up the
 * array's address itself, which is not a stream operation).
 */
#define TRN_ATTN_NOALLOC_SCRATCH_BYTES (8u << 20)
int trn_attn_fwd_noalloc_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                             void* o, float* lse, const void* gamma_q,
                             const float* noise, float* lse_pert, void* stream);

/*
 * Per-key column statistics of the attention probabilities, given the row normalisers from
 * trn_attn_fwd_f16:   p_ij = exp(t_ij - lse_i),  out_sum[j] = sum_i p_ij,
 * out_sumsq[j] = sum_i p_ij^2, over the queries i that can see key j.
 *   noise == NULL : t = scale*QK^T, lse = plain row LSE           (RoCo, ref_rms.py:274-275)
 *   noise != NULL : t = (scale*QK^T + noise)/tau, lse = lse_pert  (KeyFormer, ref_rms.py:172-174,
 *                   summed over queries as the generated kernel's C_out is,
 *                   keyformer_llama_benchmark.py:79)
 * out_sum, out_sumsq (nullable): float [batch, n_q_heads, seq_kv] contiguous.  Deterministic
 * (one workgroup owns a column block; no atomics).  v/o strides of desc are ignored; desc->q_norm
 * must be 0 (TRN_E_UNSUPPORTED otherwise).
 */
int trn_attn_colstats_f16(const trn_attn_desc* desc, const void* q, const void* k,
                          const float* lse, const float* noise,
                          float* out_sum, float* out_sumsq, void* stream);

/*
 * RoCo's statistics as mean and standard deviation (the per-key column mean and std of the attention
 * probabilities): out_mean[j] = (1/n_j) sum_i p_ij and out_std[j] = sqrt((1/n_j) sum_i p_ij^2 - out_mean[j]^2), the
 * population standard deviation, over the n_j queries that can see key j (all seq_q of them without a mask;
 * seq_q - max(0, j - (seq_kv - seq_q)) under a causal mask).  The reference defines the two sums only
 * (ref_rms.py:274-275); these are formed from them in the same kernel's epilogue.  Arguments as
 * trn_attn_colstats_f16 without noise; both outputs are required.
 */
int trn_attn_colmeanstd_f16(const trn_attn_desc* desc, const void* q, const void* k,
                            const float* lse, float* out_mean, float* out_std, void* stream);

/*
 * trn_attn_fwd_f16 and trn_attn_colstats_f16 in one call: the attention output plus the per-key statistics of its
 * probabilities -- of the perturbed probabilities when noise is given -- i.e. what one forward of the reference's
 * KeyFormer (ref_rms.py:147-179, C_out of keyformer_llama_benchmark.py:79) or RoCo (ref_rms.py:249-280) computes.
 * With at most 32 queries per head (the reference's decode-append problem) the statistics are a second sweep over
 * the keys inside the attention kernel -- one launch; otherwise the two kernels are launched one after the other,
 * and lse (lse_pert with noise) is required as the buffer that carries the row normalisers between them.
 * q_norm is not supported here.  out_sum / out_sumsq as in trn_attn_colstats_f16 (one of them may be NULL).
 */
int trn_attn_fwd_stats_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                           void* o, float* lse, const void* gamma_q,
                           const float* noise, float* lse_pert,
                           float* out_sum, float* out_sumsq, void* stream);

/*
 * trn_attn_fwd_stats_f16 with a workspace, for few queries and few heads on a LONG cache: the reference's KeyFormer
 * and RoCo classes take any prefix length P (ref_rms.py:147-179, 249-280), and one workgroup per head sweeping tens
 * of thousands of keys leaves most of the chip idle.  trn_attn_stats_workspace_bytes(desc) says for which problems
 * the library would rather split (at most 32 queries per head, heads x head_dim at most 2048, and at least 8 keys per
 * unit of that product -- 8192 keys for 8 heads of 128, 16384 for 16 -- but never fewer than 4096) and how many bytes
 * that takes, 0 otherwise.  Given a zero-initialised workspace of at least
 * that many bytes (256-byte aligned, as for trn_attn_fwd_ws_f16) the attention runs with its keys split over
 * workgroups, and the statistics -- which need the merged row normalisers -- follow as a second launch over all keys
 * at once; lse (lse_pert with noise) is then required as the buffer that carries the normalisers between the two.
 * Without a workspace, with one that is too small, without that buffer, or for a problem that would not be split,
 * the call is trn_attn_fwd_stats_f16.  Results as trn_attn_fwd_stats_f16 to the stated tolerances (the shares are
 * merged in a fixed order: the result does not depend on the run).  Neither has a counterpart in the reference, whose
 * generated kernels load the whole key axis in one tile (TritonGen.py:2474-2547).
 */
int64_t trn_attn_stats_workspace_bytes(const trn_attn_desc* desc);
int trn_attn_fwd_stats_ws_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                              void* o, float* lse, const void* gamma_q,
                              const float* noise, float* lse_pert,
                              float* out_sum, float* out_sumsq,
                              void* workspace, int64_t workspace_bytes, void* stream);

/*
 * trn_attn_fwd_stats_f16 with the noise and the statistics in fp16, for the reference's decode-append problem
 * (seq_q <= 32; TRN_E_UNSUPPORTED otherwise): its drivers allocate every tensor as fp16 -- C_out, C_out1, C_out2
 * (vanilla_llama_benchmark.py:131-139) and the noise (convert_eval_rms.py:201) -- and this entry point takes them as
 * they are, one launch, no widened copy of the noise and no narrowing copy of the scores.
 *   noise       nullable fp16 [batch, n_q_heads, seq_q, seq_kv]; the strides in desc count fp16 elements; base and
 *               pitches multiples of 8 bytes (seq_kv itself may be anything: pad the rows).
 *   out_sum, out_sumsq   fp16 [batch, n_q_heads, seq_kv] contiguous (one may be NULL): the fp32 sums of
 *               trn_attn_fwd_stats_f16 rounded to nearest once.
 */
int trn_attn_fwd_stats_half_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                                void* o, float* lse, const void* gamma_q,
                                const void* noise, float* lse_pert,
                                void* out_sum, void* out_sumsq, void* stream);

/*
 * The decode-append form of KeyFormer as its reference class returns it (ref_rms.py:171-179): the attention output
 * and the UN-REDUCED probabilities  out_probs[b,h,i,j] = softmax_j((scale*QK^T + noise)/tau)  (plain softmax(scale*QK^T)
 * when noise is NULL), float [batch, n_q_heads, seq_q, seq_kv] contiguous, masked entries 0; optionally their sums
 * over the queries as well (out_sum, nullable, as trn_attn_fwd_stats_f16).  One launch.  For decode shapes only:
 * seq_q <= 32, otherwise TRN_E_UNSUPPORTED (at prefill sizes the matrix is what these kernels exist to avoid).
 * lse / lse_pert as in trn_attn_fwd_f16 (lse_pert required with noise).
 */
int trn_attn_fwd_probs_f16(const trn_attn_desc* desc, const void* q, const void* k, const void* v,
                           void* o, float* lse, const float* noise, float* lse_pert,
                           float* out_probs, float* out_sum /* nullable */, void* stream);

/*
 * Fused RMSNorm + Q/K/V projection:  Xn = RMSNorm(X; gamma, eps);  Q = Xn Wq, K = Xn Wk,
 * V = Xn Wv  (X @ W, W is [hidden, n_out] row-major -- ref_rms.py:105-107, and the per-head
 * column slices of convert_eval_rms.py:132-138).  The row mean-square is reduced inside the
 * GEMM from the X tiles it streams, and applied as a row scale on the fp32 accumulator.
 * norm == 0 skips the normalisation (ref_rms.py:47-49).
 *
 * Each output is written "head-split": element (token t, column n) of projection P goes to
 *     P + (n / head_dim) * p_stride_h + t * p_stride_s + (n % head_dim)
 * so the same call can write token-major [T, H*D] (stride_h = head_dim, stride_s = H*D),
 * head-major [H, T, D], or rows P.. of a [H, P+M, D] KV cache (ref_rms.py:72-73).
 * hidden, n_q, n_kv multiples of 8; head_dim a multiple of 8.
 */
int trn_prenorm_qkv_f16(const void* x, const void* gamma /* nullable */,
                        const void* wq, const void* wk, const void* wv,
                        void* q, void* k, void* v,
                        int64_t tokens, int64_t hidden, int64_t n_q, int64_t n_kv, int64_t head_dim,
                        int64_t ldx, int64_t ldwq, int64_t ldwk, int64_t ldwv,
                        int64_t q_stride_h, int64_t q_stride_s,
                        int64_t k_stride_h, int64_t k_stride_s,
                        int64_t v_stride_h, int64_t v_stride_s,
                        float eps, int32_t norm, void* stream);

/*
 * Up to three plain projections of one activation matrix:  out_i = x w_i (+ addend_i),  i < n_mats <= 3, with
 * x [tokens, hidden], w_i [hidden, n_i], out_i / addend_i [tokens, n_i], all fp16 row-major with the given row
 * pitches; addend (the array or an entry) may be NULL, and addend_i may be out_i itself.  The product is rounded to
 * fp16 before the addend is added, as two separate GEMMs would leave it.  These are the building blocks of the
 * reference's other two TritonGen workloads: LoRA, O = X W + (X A) B (lora_benchmark.py:41-53: X [M,N], W [N,P],
 * A [N,R], B [R,P], intermediates C = X W, D = X A, E = D B) as  {O, D} = X {W, A};  O = D B + O;  and the gated MLP
 * (gmlp_benchmark.py:53-64: X [M,K], W1, W2 [K,N], intermediates C1, C1_exp, C2) as  {C1, C2} = X {W1, W2}  followed
 * by trn_gate_f16.  Same kernels and tile selection as trn_prenorm_qkv_f16 (norm off).  hidden, n_i multiples of 8.
 */
int trn_linear_f16(const void* x, int64_t tokens, int64_t hidden, int64_t ldx, int32_t n_mats,
                   const void* const* w, const int64_t* n, const int64_t* ldw,
                   void* const* out, const int64_t* ldo, const void* const* addend /* nullable */, void* stream);

/*
 * Gate of the gated MLP, elementwise over [rows, cols] fp16:  out = sigmoid(c1) * c2  (kind 0)  or
 * out = c1 * sigmoid(c1) * c2  (kind 1, SiLU).  The reference names the tensors (gmlp_benchmark.py:53-64) and has a
 * sigmoid operator (NodeType.py:21); the IR that combines them is not in its tree, so both common gates are offered.
 * cols a multiple of 8; out may alias c1 or c2.
 */
int trn_gate_f16(const void* c1, const void* c2, void* out, int64_t rows, int64_t cols,
                 int64_t ld1, int64_t ld2, int64_t ldo, int32_t kind, void* stream);

/*
 * Measurement aid, no counterpart in the reference: the name (as a profiler's kernel trace prints it) of the kernel
 * instantiation that trn_attn_fwd_f16 launches for this problem -- decided by the same rules as the launch itself,
 * so that a benchmark can say which kernel its timing belongs to.  with_noise: as if a noise tensor were passed.
 * It speaks for trn_attn_fwd_f16 only: fp32 noise, no workspace.  With at most 32 queries per head the other entry
 * points launch the same kernel template with other last arguments -- fp16 noise (trn_attn_fwd_stats_half_f16) shows
 * as <..., 2> where this function says <..., 1>, and a workspace that splits the keys turns the column shares
 * (the middle argument) back to 1.  Returns "" for an invalid descriptor.  The string is static.
 */
const char* trn_attn_fwd_kernel_name(const trn_attn_desc* desc, int32_t with_noise);

/*
 * Measurement aid, no counterpart in the reference: a plain 16-bytes-per-lane streaming copy of `bytes`
 * (a multiple of 16) from src to dst.  bench.py and the profiling recipes run it on a buffer of known size so
 * that HBM byte counters (FETCH_SIZE / WRITE_SIZE) and achieved GB/s of the real kernels can be scaled
 * against a kernel whose traffic is known exactly.
 */
int trn_calibration_copy(const void* src, void* dst, int64_t bytes, void* stream);

/*
 * Measurement aid, no counterpart in the reference: n_workgroups x 256 threads each issue
 * iters x 8 back-to-back v_mfma_f32_32x32x16_f16 (n_workgroups*4*iters*8*32768 flop in all) on register
 * operands read once from `operands` (fp16, >= 65536 bytes; its data pattern sets the switching activity)
 * and write a checksum to `sink` (>= n_workgroups*256 floats).  Run with all-zero and with random operands it
 * shows the nominal and the power-limited sustained MFMA rate of the board, the latter being the practical
 * ceiling for MFMA-bound kernels on real data.
 */
int trn_calibration_mfma(const void* operands, float* sink, int32_t iters, int32_t n_workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRINITY_HIP_H */
