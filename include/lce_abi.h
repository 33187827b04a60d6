/* C ABI of liblce_gfx950.so: fused lm-head linear + log-prob + entropy for MI355X (gfx950).
 *
 * Plain pointers and sizes only; every buffer is owned by the caller and lives in device memory
 * of the current HIP device; every call is asynchronous on `stream` (a hipStream_t passed as
 * void*) and allocates nothing.  All functions return 0 on success or a negative LCE_E_* code and
 * never throw; lce_last_error() gives the text of the calling thread's last failure.
 *
 * Each entry point names the reference interface it stands in for (paths relative to the
 * reference tree).  The reference has no native ABI of its own (its kernels are Triton), so what
 * is replaced are its Python host launchers.
 */
#ifndef LCE_ABI_H
#define LCE_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LCE_ABI_VERSION 10

enum { LCE_DTYPE_BF16 = 0, LCE_DTYPE_F32 = 1, LCE_DTYPE_F16 = 2 };
enum { LCE_REDUCTION_NONE = 0, LCE_REDUCTION_SUM = 1, LCE_REDUCTION_MEAN = 2 }; /* verl/utils/kernel/kernels.py:102-126 */
enum {
  LCE_OK = 0,
  LCE_E_ARG = -1,       /* bad shape, dtype, alignment or null pointer */
  LCE_E_WORKSPACE = -2, /* workspace too small */
  LCE_E_LAUNCH = -3,    /* HIP reported an error at launch */
  LCE_E_BUSY = -4       /* lce_forward_static: the built-in scratch buffer is still in use by a call on another stream */
};

int lce_abi_version(void);
const char* lce_last_error(void);

/* Forward.  Replaces efficient_entropy_forward (verl/utils/kernel/kernels.py:569-759) and the two
 * Triton kernels it launches (:186-349 mainloop, :352-441 epilogue).
 *   hidden [T, H] row stride ldh, weight [V, H] row stride ldw (elements; K-contiguous), dtype LCE_DTYPE_*
 *   labels [T] int64, values outside [0, V) give logprob = -logsumexp (no label logit)
 *   logits = (hidden . weight^T) * (1 / temperature), accumulated in fp32, never written to memory
 * Outputs, all fp32:
 *   logprobs [T] (reduction none) or [1] (sum / mean over tokens); entropy [T];
 *   maximum [T], accumulate [T], entropy_b [T]: per-token max logit, sum exp(logit - max) and
 *   sum softmax * logit, kept for the backward.
 * H must be a multiple of 64 (bf16) / 32 (fp32); pointers 16-byte aligned; ldh, ldw multiples of
 * 8 (bf16) / 4 (fp32) elements and below 16 MiB per row (256 rows are addressed with 32-bit offsets). */
size_t lce_forward_workspace_bytes(int64_t T, int64_t H, int64_t V, int dtype);
int lce_forward(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                int64_t H, int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy,
                float* maximum, float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes,
                void* stream);

/* The same forward for callers that cannot allocate device memory and have no workspace to hand over (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The
 * partial statistics go to a buffer of LCE_STATIC_SCRATCH_BYTES that is part of the library's own device image (one
 * copy per GPU, held until the process ends); the call allocates nothing, uses at most as many vocabulary splits as the
 * buffer has room for (so its results may differ from lce_forward's in the last bits of the fp32 sums) and returns
 * LCE_E_WORKSPACE when there is no room for four (beyond about 116000 tokens).  All calls on one GPU share the
 * buffer, so calls that overlap on one GPU would race for it; calls on one stream do not overlap.  The library keeps, per
 * GPU, the stream of the last call and an event behind its last kernel: a call on another stream while that one has not
 * finished returns LCE_E_BUSY and launches nothing (host-side check, no device work).  Calls recorded into a HIP graph
 * are neither checked nor remembered: the order of a graph's nodes is the caller's.  The first call on a device looks
 * the buffer's address up and creates that event, so make one call outside a graph capture before capturing; with
 * lce_profile_enable(1) every call also creates timing events. */
#define LCE_STATIC_SCRATCH_BYTES (8u << 20)
int lce_forward_static(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T, int64_t H,
                       int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy, float* maximum,
                       float* accumulate, float* entropy_b, void* stream);

/* Backward.  Replaces efficient_entropy_backward (verl/utils/kernel/kernels.py:1518-1729): its
 * d_logits kernel (:1380-1515) and the two vendor GEMMs per vocab split (:1714-1724).
 *   dlogprobs [T] fp32 (reduction none) or [1] fp32 (sum / mean); dentropy [T] fp32 or NULL (treated as zero)
 *   d_hidden [T, H] and d_weight [V, H], contiguous, in the input dtype.  One of the two may be NULL (the reference
 *   always computes both): that gradient is not wanted, e.g. d_weight for a frozen lm-head, and its GEMM, a third
 *   of the backward's work, is left out; the other gradient is bit for bit what the full call gives.
 * The vocabulary is processed in chunks of `vchunk` columns (0 = library default, else a multiple
 * of 256); per chunk the gradient of the logits exists only as a [T, vchunk] tile pair in the
 * workspace.  Sums over the vocabulary (d_hidden) and over tokens (d_weight) are carried in fp32
 * and rounded once. */
size_t lce_backward_workspace_bytes(int64_t T, int64_t H, int64_t V, int dtype, int64_t vchunk);
int lce_backward(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                 int64_t H, int64_t V, int dtype, float temperature, int reduction, const float* maximum,
                 const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                 void* d_hidden, void* d_weight, void* workspace, size_t workspace_bytes, int64_t vchunk,
                 void* stream);

/* The same backward with both gradients returned in fp32, d_hidden [T, H] and d_weight [V, H] contiguous: what
 * should_return_fp32_grad of efficient_entropy_backward asks for (verl/utils/kernel/kernels.py:1562-1567).  The sums are
 * carried in fp32 anyway; here they are stored without the final rounding to the input dtype.  Same workspace. */
int lce_backward_f32(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T, int64_t H,
                     int64_t V, int dtype, float temperature, int reduction, const float* maximum, const float* accumulate,
                     const float* entropy_b, const float* dlogprobs, const float* dentropy, float* d_hidden, float* d_weight,
                     void* workspace, size_t workspace_bytes, int64_t vchunk, void* stream);

/* The pair above with the logits kept between the two calls, the way autograd keeps any activation, while they are no
 * larger than the weight they came from.  The reference's backward recomputes the logits from hidden and weight
 * (verl/utils/kernel/kernels.py:1380-1515), which is what keeps [T, V] out of memory when T is large, and what lce_backward
 * does.  With few tokens [T, V] in fp32 is a fraction of the weight itself (T * V * 4 against V * H * 2 bytes: 4 % at 64
 * tokens and H=3584, 57 % at 1024), and keeping it saves the backward its pass over the weight and its T x V x H product
 * for the logits (64 tokens, H=3584, V=152064: 39 MB kept, 1.09 GB not read; 1024 tokens: a quarter of the matrix work).
 *   lce_logits_cache_max_tokens: the largest T for which a cache is offered: H / 2 for 16-bit inputs (the
 *     cache never exceeds the weight), or LCE_OPT_KEEP_LOGITS_TOKENS where that is lower; 0 for fp32 inputs and under diagnostic settings that force a tile variant.
 *   lce_logits_cache_bytes: size of the buffer for this shape, or 0 when T is beyond that: then pass NULL below.
 *   lce_forward_keep_logits: lce_forward; with logits_cache != NULL it also writes hidden . weight^T there in fp32
 *     (private layout).  Same outputs, bit for bit.
 *   lce_backward_from_logits: lce_backward (grads_fp32 = 0) or lce_backward_f32 (grads_fp32 = 1; d_hidden, d_weight are
 *     float* then); with logits_cache != NULL, as written by lce_forward_keep_logits for the same hidden, weight, T, H, V
 *     and dtype, the gradient of the logits is computed from it with the same expressions, so both gradients are bit for
 *     bit those of lce_backward.  The cache is only read. */
int64_t lce_logits_cache_max_tokens(int64_t H, int dtype);
size_t lce_logits_cache_bytes(int64_t T, int64_t H, int64_t V, int dtype);
int lce_forward_keep_logits(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                            int64_t H, int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy,
                            float* maximum, float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes,
                            void* logits_cache, size_t logits_cache_bytes, void* stream);
int lce_backward_from_logits(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                             int64_t H, int64_t V, int dtype, float temperature, int reduction, const float* maximum,
                             const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                             void* d_hidden, void* d_weight, int grads_fp32, void* workspace, size_t workspace_bytes, int64_t vchunk,
                             const void* logits_cache, size_t logits_cache_bytes, void* stream);

/* Vocabulary-parallel building blocks: what one rank of a tensor-parallel lm-head runs on its shard
 * W[vocab_offset : vocab_offset + V_local, :] of the vocabulary.  The exchange between the ranks (an
 * all-gather of the partials, a sum of d_hidden) is the caller's.  Replaces the per-rank part of the
 * reference's tensor-parallel branch: the mainloop matching labels against `rank * vocab_size`
 * (verl/utils/kernel/kernels.py:328, :343-344), its all-reduced statistics and TP epilogue (:444-566, :705-757)
 * and the backward's label mask with the same offset (:1503).  labels are GLOBAL vocabulary ids.
 *   lce_forward_shard: partials [T, 4] fp32 = per token (max logit, sum exp(logit - max),
 *     sum logit * exp(logit - max), label logit or 0 if the label is not in the shard), logits = h.w / temperature.
 *     Workspace as lce_forward_workspace_bytes(T, H, V_local, dtype).
 *   lce_merge_shards: partials [R, T, 4] (shard-major, e.g. straight out of an all-gather) -> the five outputs of
 *     lce_forward for the whole vocabulary, merged in the fixed order r = 0..R-1.  Workspace: 4*T bytes for
 *     reduction sum / mean, else unused.
 *   lce_backward_shard: as lce_backward with the merged statistics; d_weight_shard [V_local, H] is complete,
 *     d_hidden_partial [T, H] is this shard's contribution (the ranks' partials add up to d_hidden).
 *     Workspace as lce_backward_workspace_bytes(T, H, V_local, dtype, vchunk). */
int lce_forward_shard(const void* hidden, int64_t ldh, const void* weight_shard, int64_t ldw, const int64_t* labels, int64_t T,
                      int64_t H, int64_t V_local, int64_t vocab_offset, int dtype, float temperature, float* partials,
                      void* workspace, size_t workspace_bytes, void* stream);
int lce_merge_shards(const float* partials, int R, int64_t T, int reduction, float* logprobs, float* entropy, float* maximum,
                     float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes, void* stream);
int lce_backward_shard(const void* hidden, int64_t ldh, const void* weight_shard, int64_t ldw, const int64_t* labels, int64_t T,
                       int64_t H, int64_t V_local, int64_t vocab_offset, int dtype, float temperature, int reduction,
                       const float* maximum, const float* accumulate, const float* entropy_b, const float* dlogprobs,
                       const float* dentropy, void* d_hidden_partial, void* d_weight_shard, void* workspace,
                       size_t workspace_bytes, int64_t vchunk, void* stream);

/* Unfused twins on logits that already exist in memory.
 * Replaces logprobs_from_logits (verl/utils/torch_functional.py:73-107, :155-207) and
 * entropy_from_logits (:231-245) with one pass over the rows.
 *   logits [R, V] row stride ldl, dtype LCE_DTYPE_*; labels [R] int64 or NULL; logprobs / entropy [R] fp32, either may be NULL;
 *   stats [R, 2] fp32 or NULL: per row logsumexp and sum softmax * logit, which let the backward skip its own reduction pass. */
int lce_logits_forward(const void* logits, int64_t ldl, const int64_t* labels, int64_t R, int64_t V, int dtype,
                       float* logprobs, float* entropy, float* stats, void* stream);
/* d_logits [R, V] (row stride ldd, same dtype as logits) of sum(dlogprobs*logprobs) + sum(dentropy*entropy);
 * dlogprobs / dentropy [R] fp32, either may be NULL; stats as written by lce_logits_forward for the same logits, or NULL
 * (then recomputed).  Autograd twin of the two functions above. */
int lce_logits_backward(const void* logits, int64_t ldl, const int64_t* labels, int64_t R, int64_t V, int dtype,
                        const float* stats, const float* dlogprobs, const float* dentropy, void* d_logits, int64_t ldd,
                        void* stream);

/* Replaces calculate_sum_pi_squared_from_logits (verl/utils/torch_functional.py:687-703; called on the actor's
 * logits at verl/workers/engine/fsdp/transformer_impl.py:1413,1513): out[r] = sum_v softmax(logits[r])_v ^ 2
 * = exp(logsumexp(2 z) - 2 logsumexp(z)), one pass over the row, fp32 arithmetic.  logits [R, V] row stride ldl;
 * out [R] fp32; lse_out [R] fp32 or NULL: the rows' logsumexp, which lets the backward skip its own reduction pass. */
int lce_logits_sum_pi_squared(const void* logits, int64_t ldl, int64_t R, int64_t V, int dtype, float* out, float* lse_out,
                              void* stream);
/* Its autograd twin (the reference's function is plain torch, hence differentiable): d_logits [R, V] (row stride ldd, dtype
 * of the logits) = g[r] * 2 p (p - S_r), p = softmax(logits[r]), S_r = sum_v p_v^2.  g [R] fp32; lse / sum_pi2 [R] fp32 as
 * the forward wrote them, or NULL (then both are recomputed from the row).  One read and one write of the rows. */
int lce_logits_sum_pi_squared_backward(const void* logits, int64_t ldl, int64_t R, int64_t V, int dtype, const float* lse,
                                       const float* sum_pi2, const float* g, void* d_logits, int64_t ldd, void* stream);

/* Consumer of the path's outputs: the clipped PPO policy loss with dual clip, any of agg_loss's aggregation
 * modes, the entropy bonus and the KL penalty against a reference policy.  Replaces, for the vanilla loss,
 * compute_policy_loss_vanilla + agg_loss (verl/trainer/ppo/core_algos.py:1140-1206, :1286-1376), kl_penalty
 * (:2188-2251) and the entropy and KL terms of ppo_loss (verl/workers/utils/losses.py:134-153), and yields the
 * upstream gradients lce_backward consumes, so no elementwise autograd graph sits between the two kernels.
 *   all inputs fp32 [rows, row_len] contiguous (batch x response; rows = 1 for a flat token list, which the
 *   token modes treat alike); entropy / g_entropy may both be NULL; is_weights (rollout correction factor on
 *   the policy loss, core_algos.py:1362-1363, a constant w.r.t. the gradients) may be NULL
 *   kl_type LCE_PPO_KL_* (K1 "kl", ABS "abs", K2 "mse", K3 "low_var_kl"), optionally | LCE_PPO_KL_STRAIGHT_THROUGH
 *   (the reference's "+" suffix: the estimator's value with k2's gradient); needs ref_log_prob; adds
 *   kl_coef * agg(kl) to the loss
 *   log_prob == NULL (then old_log_prob, advantages are ignored, g_log_prob is NULL, no KL): the call is agg_loss
 *   applied to `entropy`; with entropy_coeff = -1, out[0] = agg(entropy) and g_entropy is its gradient
 *   agg_mode LCE_PPO_*: per row r with n_r = sum(mask_r), a token of row r weighs
 *     TOKEN_MEAN dp_size / batch_num_tokens; TOKEN_SUM dp_size; SEQ_MEAN_TOKEN_SUM dp_size / global_batch_size;
 *     SEQ_MEAN_TOKEN_SUM_NORM that / loss_scale_factor; SEQ_MEAN_TOKEN_MEAN dp_size / global_batch_size / (n_r + 1e-8);
 *     the SEQ modes skip rows with n_r = 0
 *   batch_num_tokens <= 0: sum(mask); global_batch_size <= 0: number of rows with n_r > 0;
 *   loss_scale_factor <= 0: row_len
 *   out [16]: loss, pg_loss, entropy_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower, sum(mask), the mode's common
 *   factor, kl_loss; the rest is reserved
 *   g_log_prob, g_entropy [rows, row_len]: d loss / d log_prob, d loss / d entropy (zero outside the mask) */
enum { LCE_PPO_TOKEN_MEAN = 0, LCE_PPO_TOKEN_SUM = 1, LCE_PPO_SEQ_MEAN_TOKEN_SUM = 2,
       LCE_PPO_SEQ_MEAN_TOKEN_SUM_NORM = 3, LCE_PPO_SEQ_MEAN_TOKEN_MEAN = 4 };
enum { LCE_PPO_KL_NONE = 0, LCE_PPO_KL_K1 = 1, LCE_PPO_KL_ABS = 2, LCE_PPO_KL_K2 = 3, LCE_PPO_KL_K3 = 4,
       LCE_PPO_KL_STRAIGHT_THROUGH = 16 };
size_t lce_ppo_loss_workspace_bytes(int64_t rows, int64_t row_len);
int lce_ppo_loss(const float* log_prob, const float* entropy, const float* old_log_prob, const float* advantages,
                 const float* mask, const float* is_weights, const float* ref_log_prob, int kl_type, float kl_coef,
                 int64_t rows, int64_t row_len, int agg_mode,
                 float clip_low, float clip_high, float clip_c, float entropy_coeff, float dp_size,
                 float batch_num_tokens, float global_batch_size, float loss_scale_factor, float* out,
                 float* g_log_prob, float* g_entropy, void* workspace, size_t workspace_bytes, void* stream);

/* The same loss on PACKED model outputs: folds in the response slice that the no-padding engines apply between the
 * head and the loss, no_padding_2_padding (verl/workers/utils/padding.py:97-141): for sequence r with prompt length
 * P_r > 0 and response length R_r, packed end offset E_r = sum_{q <= r} (P_q + R_q), the padded element (r, c) is
 * log_prob_packed[E_r - R_r - 1 + c] for c < R_r (the model output left-shifted by one token) and 0 beyond.
 *   log_prob_packed, entropy_packed (may be NULL with g_entropy_packed) [total_nnz] fp32: what the fused head returns
 *   response_start [rows] int64 = E_r - R_r - 1, response_len [rows] int64 = R_r (0 allowed), both on the device
 *   everything else as in lce_ppo_loss, [rows, row_len] with row_len = max_response_len
 *   g_log_prob_packed, g_entropy_packed [total_nnz]: the gradients IN PACKED ORDER (zero at every position that no
 *   response token maps to), i.e. exactly the dlogprobs / dentropy vectors lce_backward takes: no gather or scatter
 *   of per-token data remains between the two kernels. */
int lce_ppo_loss_packed(const float* log_prob_packed, const float* entropy_packed, int64_t total_nnz, const int64_t* response_start,
                        const int64_t* response_len, const float* old_log_prob, const float* advantages, const float* mask,
                        const float* is_weights, const float* ref_log_prob, int kl_type, float kl_coef, int64_t rows, int64_t row_len,
                        int agg_mode, float clip_low, float clip_high, float clip_c, float entropy_coeff, float dp_size,
                        float batch_num_tokens, float global_batch_size, float loss_scale_factor, float* out,
                        float* g_log_prob_packed, float* g_entropy_packed, void* workspace, size_t workspace_bytes, void* stream);

/* Product-level options (process-wide; every entry point works from one snapshot of the settings taken when it starts).
 * LCE_OPT_WORKSPACE_BUDGET (default 0 = the built-in rule, chunks of 8192 vocabulary columns or wider while one
 * d_logits buffer stays within 256 MiB): a byte count; lce_backward_workspace_bytes with vocab_chunk <= 0 then
 * returns the workspace of the widest chunk that fits it (never below 2048 columns, never above the bound
 * 0.25 * T * V * esz + 4 * V * H), and lce_backward with vocab_chunk <= 0 uses that chunk.  An explicit vocab_chunk
 * is not touched.  Takes the role of the reference's fixed vocab_per_split = 9504 (verl/utils/kernel/kernels.py:1666-1670).
 * LCE_OPT_LABEL_TERM_OUTSIDE (default 2, 16-bit inputs only) chooses the data format of the gradient of the logits:
 * 0 = the label's entry is rounded to 16 bits with the rest of the d_logits tile, which is the reference's format
 * (verl/utils/kernel/kernels.py:1666-1724); 1 = its one-hot part g_logprob / temperature * 1[v == label] is added to
 * d_hidden and to the label rows of d_weight in fp32 instead; 2 = the label's whole entry (one-hot and softmax part,
 * with hidden . W[label] recomputed per token) is kept out of the tiles and added in fp32.  Changes the workspace size:
 * set it before querying lce_backward_workspace_bytes.
 * LCE_OPT_KEEP_LOGITS_TOKENS (default LCE_KEEP_LOGITS_NO_LIMIT; any count >= 0): the token count up to which
 * lce_logits_cache_bytes offers a cache, next to its own bound of H / 2 tokens; 0 makes every backward recompute its
 * logits, as the reference does at every size. */
#define LCE_KEEP_LOGITS_NO_LIMIT ((int64_t)1 << 40)
enum {
  LCE_OPT_LABEL_TERM_OUTSIDE = 4,
  LCE_OPT_WORKSPACE_BUDGET = 8,
  LCE_OPT_KEEP_LOGITS_TOKENS = 11
};
int lce_set_option(int key, int64_t value);

/* ---------------------------------------------------------------------------------------------------------------------
 * DIAGNOSTIC BLOCK (block version 2).  Nothing below is needed to use the path; none of it has a counterpart in the
 * reference.  It exists so that the benchmark and the tests can time the pieces of a call separately and run the
 * mainloops on their own.  A caller that integrates the library binds the entry points above and ignores these.
 * ------------------------------------------------------------------------------------------------------------------- */

/* C[M, N] (fp32, row stride ldc) = A[M, K] . B[N, K]^T with one of the library's MFMA mainloops (the same code that the
 * entry points above run).  K a multiple of 64 (16-bit) / 32 (fp32).  variant: see lce_set_variant. */
int lce_gemm_nt(const void* A, int64_t lda, const void* B, int64_t ldb, float* C, int64_t ldc, int64_t M, int64_t N,
                int64_t K, int dtype, int variant, void* stream);
/* Twin for K-major operands (bf16 only): C[M, N] = A[K, M]^T . B[K, N], the layout of the d_weight GEMM
 * (A = d_logits [tokens, vocab], B = hidden [tokens, H]).  K a multiple of 64; lda >= M and ldb >= N rounded up to 256.
 * variant 3 runs the four-wave 16x16x32 loop, any other the eight-wave split ring. */
int lce_gemm_tn(const void* A, int64_t lda, const void* B, int64_t ldb, float* C, int64_t ldc, int64_t M, int64_t N, int64_t K,
                int variant, void* stream);

/* Forces one mainloop for forward and backward instead of the choice by size, 0 <= variant < lce_num_variants();
 * -1 restores the defaults.  0, 1: eight waves of 64 x 128 on v_mfma_f32_32x32x16, LDS ring of five half slabs with the
 * A resp. B operand fetched early; 2: the same tile with a ring of two whole slabs; 3: four waves of 128 x 128 on
 * v_mfma_f32_16x16x32 (16-bit inputs; fp32 inputs run variant 1's loop on v_mfma_f32_32x32x2).  The backward is built on
 * variants 1 and 3: forcing 0 or 2 leaves it on 1. */
int lce_set_variant(int variant);
int lce_num_variants(void);
/* Diagnostic keys of lce_set_option.  LCE_OPT_SPLIT_BACKWARD_LAUNCHES: launch the d_logits tiles and the two gradient
 * GEMMs of a backward chunk as three kernels instead of one (per-phase timing).  LCE_OPT_DLOGITS_TOKENS_FIRST: order in
 * which an XCD's consecutive blocks of d_logits tiles walk the chunk: -1 = chosen by size (default), 0 = along the
 * vocabulary, 1 = along the tokens.  LCE_OPT_DHIDDEN_KSPLIT (default 0 = by shape): K slices of the d_hidden GEMM, each
 * with its own fp32 partial that is summed in a fixed order afterwards (0..16; changes the workspace size).
 * LCE_OPT_FEW_TOKEN_GEMMS (default 1, 16-bit inputs): with at most 128 tokens both gradient GEMMs of the backward run
 * as one launch of streaming kernels; 0 = the 256 x 256 tile kernels, which the tests compare them with (changes the
 * workspace size). */
enum {
  LCE_OPT_SPLIT_BACKWARD_LAUNCHES = 1,
  LCE_OPT_DLOGITS_TOKENS_FIRST = 2,
  LCE_OPT_DHIDDEN_KSPLIT = 7,
  LCE_OPT_FEW_TOKEN_GEMMS = 9
};

/* Per-kernel timing for benchmarks.  While enabled, every kernel launch of the library is bracketed by HIP events on the
 * caller's stream; lce_profile_read waits for them and returns, per kernel class c < lce_profile_num_classes(), the
 * summed duration in milliseconds and the number of launches (arrays sized by the caller).  Creating events allocates
 * host-side driver objects (also inside lce_forward_static), so keep it disabled under graph capture. */
int lce_profile_enable(int on);
int lce_profile_num_classes(void);
const char* lce_profile_class_name(int cls);
int lce_profile_read(double* total_ms, int64_t* launches, int reset);

#ifdef __cplusplus
}
#endif
#endif /* LCE_ABI_H */
