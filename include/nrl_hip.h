/*
 * nrl_hip.h - C ABI of librl_amd_hip.so: the GRPO logits -> logprob -> loss hot path
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - every entry point enqueues work on `stream` (a hipStream_t passed as void*) and returns
 *     without synchronising; nothing is allocated or freed inside the library;
 *   - sizes and strides are in ELEMENTS (not bytes); the vocabulary axis is contiguous;
 *   - return value: 0 = ok, negative = NRL_E_* below; nrl_last_error() gives the text for the
 *     calling thread;
 *   - the library keeps no state between calls: entry points may be called from any host
 *     thread (forward pass and autograd thread alike).  The one exception is
 *     nrl_grpo_loss_fwd_bwd_static, which owns a fixed device array (see there).
 *
 * The reference (NVIDIA NeMo-RL) has no FFI; each entry point names the Python code whose
 * arithmetic it replaces (paths relative to the reference tree).
 */
#ifndef NRL_HIP_H
#define NRL_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NRL_OK 0
#define NRL_E_INVALID (-1)     /* bad argument (shape, stride, dtype, null pointer)   */
#define NRL_E_UNSUPPORTED (-2) /* combination not built                                */
#define NRL_E_LAUNCH (-3)      /* hipLaunchKernel / runtime error                      */
#define NRL_E_WORKSPACE (-4)   /* workspace too small                                  */

enum nrl_dtype { NRL_F32 = 0, NRL_BF16 = 1, NRL_F16 = 2 };

/* how the temperature divide is rounded (nemo_rl/models/automodel/train.py:180-194 divides the
 * logits in place in their own dtype):  DIV = round(x / T), what torch does on the CPU;
 * RCP = round(x * (1/T)) with 1/T rounded to fp32 first, what torch does on the GPU. */
enum nrl_temp_mode { NRL_TEMP_DIV = 0, NRL_TEMP_RCP = 1 };

/* changes whenever an entry point is added or a signature changes; a binding should refuse a library it was not
 * written for */
int nrl_version(void);
const char* nrl_last_error(void);

/* Row addressing shared by the logprob entry points.  Row (o, i), 0 <= o < n_outer,
 * 0 <= i < n_inner, lives at logits + o*stride_outer + i*stride_inner and has `vocab` contiguous
 * elements.  Its target id is targets[o*tgt_stride_outer + i*tgt_stride_inner].  Passing
 * targets = input_ids + 1 with n_inner = S-1 gives the reference's roll(-1) + drop-last-column
 * without materialising either. */
typedef struct nrl_rows {
    const void* logits;
    int32_t dtype; /* nrl_dtype */
    int64_t n_outer, n_inner, vocab;
    int64_t stride_outer, stride_inner;
    const int64_t* targets;
    int64_t tgt_stride_outer, tgt_stride_inner;
    int64_t vocab_start, vocab_end; /* targets outside [start, end) -> logprob 0, no one-hot */
    float temperature;              /* 1.0 = off */
    int32_t temp_mode;              /* nrl_temp_mode */
} nrl_rows;

/* K1  logits -> token logprob, one streaming pass per row (online log-sum-exp + gather).
 * Replaces DistributedLogprob.forward / ChunkedDistributedLogprob.forward
 * (nemo_rl/distributed/model_utils.py:136-165, 289-331) and the log_softmax + gather of
 * get_next_token_logprobs_from_logits (:1677-1693) at TP = CP = 1.
 * logprob_out, lse_out: fp32 [n_outer * n_inner]; lse_out may be NULL (inference_only). */
int nrl_logprob_fwd(const nrl_rows* rows, float* logprob_out, float* lse_out, void* stream);

/* Forward-only logprobs in the shape a policy worker returns for prev_logprobs / reference_policy_logprobs.
 * Replaces LogprobsPostProcessor.__call__ for right-padded batches at TP = CP = 1
 * (nemo_rl/models/automodel/train.py:689-806: _compute_local_logprobs, the prepended zero column and the
 * input_lengths mask): out[b, 0] = 0, out[b, i] = logprob(row i-1 -> target i-1) for 1 <= i < lengths[b],
 * 0 for i >= lengths[b].  rows describes the n_inner = S-1 rows per sequence exactly as for nrl_logprob_fwd;
 * lengths: int64 [n_outer] device; out: fp32 [n_outer, n_inner + 1].  Padding rows are never read. */
int nrl_logprob_post_fwd(const nrl_rows* rows, const int64_t* lengths, float* out, void* stream);

/* The stable log-softmax itself, materialised: y_v = (x_v - max) - log(sum_u exp(x_u - max)), fp32
 * arithmetic, written in the logits' dtype.  Replaces _compute_distributed_log_softmax[_with_grad]
 * (nemo_rl/distributed/model_utils.py:33-79) at TP = 1; the logprob entry points above never
 * materialise it.  Row r at logits + r*row_stride / out + r*out_row_stride (elements, unit column stride). */
int nrl_log_softmax_fwd(const void* logits, int32_t dtype, int64_t n_rows, int64_t vocab,
                        int64_t row_stride, void* out, int64_t out_row_stride, void* stream);

/* Its backward (what autograd derives from :49-67): dx_v = g_v - exp(y_v) * sum_u g_u, from the saved
 * forward output; logprobs, grad and dx share the dtype. */
int nrl_log_softmax_bwd(const void* logprobs, int32_t dtype, int64_t n_rows, int64_t vocab,
                        int64_t lp_row_stride, const void* grad, int64_t grad_row_stride, void* dx,
                        int64_t dx_row_stride, void* stream);

/* K2  dlogits = g * (onehot(target) - exp(x - lse)), written once in the logits' dtype.
 * Replaces DistributedLogprob.backward / ChunkedDistributedLogprob.backward (:167-207, 333-380).
 * grad: fp32 upstream gradient of the logprobs, element (o, i) at
 * grad[o*grad_stride_outer + i*grad_stride_inner].
 * dlogits: same dtype as the logits; row (o, i) at dlogits + o*d_stride_outer + i*d_stride_inner
 * for 0 <= i < d_n_inner; rows with i >= rows->n_inner (positions the forward dropped) are
 * zero-filled.  dlogits may alias the logits (in-place gradient).  Rows whose g is exactly 0 are
 * zero-filled without reading the logits.
 * Placement: every kernel here that reads logits and writes a tensor of the same shape streams one row in
 * and another out at a fixed distance, and HBM serves the pair up to 17 % slower when (dlogits - logits) is
 * a multiple of 512 KiB (rows of a power-of-two size) or 64 - 256 KiB past a multiple of 2 MiB (V = 151936
 * bf16).  A separate output buffer is best started about 1.69 MiB (0x1B0000) past a multiple of 2 MiB
 * relative to the logits. */
int nrl_logprob_bwd(const nrl_rows* rows, const float* lse, const float* grad,
                    int64_t grad_stride_outer, int64_t grad_stride_inner, void* dlogits,
                    int64_t d_n_inner, int64_t d_stride_outer, int64_t d_stride_inner, void* stream);

/* dst[o, i, :] = src[o, i, :] * (factor[0] / divisor), fp32 product narrowed once to `dtype`; row (o, i) at
 * base + o*stride_outer + i*stride_inner; dst may be src (in place).  `factor` is a DEVICE scalar, so the
 * caller never waits for its value; in place with factor[0] / divisor exactly 1 no row is read or written.
 * Replaces two elementwise passes of the reference:
 *   - the in-place temperature divide apply_temperature_scaling = logits.div_(T)
 *     (nemo_rl/models/automodel/train.py:180-194, nemo_rl/models/megatron/train.py:203-217) and its backward,
 *     with factor = 1 and divisor = T: x * (1 / T) with the quotient in fp32, which is how the GPU divide by a
 *     scalar rounds;
 *   - the multiplication autograd applies to a gradient when the loss was scaled after the loss function
 *     returned (automodel/train.py:547 multiplies by dp_size * cp_size, megatron/train.py:590-592 by
 *     num_microbatches / cp_size), applied to a gradient the single-pass entry points have already written. */
int nrl_scale_rows(const void* src, void* dst, int32_t dtype, int64_t n_outer, int64_t n_inner, int64_t vocab,
                   int64_t src_stride_outer, int64_t src_stride_inner, int64_t dst_stride_outer,
                   int64_t dst_stride_inner, const float* factor, float divisor, void* stream);

/* _pack_input_ids (nemo_rl/algorithms/loss/utils.py:214-261) at CP = 1, on the device and without a host read of
 * the boundaries: input_ids int64 [batch, width] rows of row_stride -> packed_out int64 [total_out].  Sequence s
 * fills [cu_seqlens_padded[s], cu_seqlens_padded[s+1]) with its first min(cu_seqlens[s+1] - cu_seqlens[s], width)
 * ids, rolled by roll_shift inside that span (element j comes from (j - roll_shift) mod span); every other
 * position, and the positions from cu_seqlens_padded[batch] to total_out, are zero.  Both boundary arrays are
 * int32 [batch + 1] on the device. */
int nrl_pack_input_ids(const int64_t* input_ids, int64_t batch, int64_t width, int64_t row_stride,
                       const int32_t* cu_seqlens, const int32_t* cu_seqlens_padded, int64_t roll_shift,
                       int64_t* packed_out, int64_t total_out, void* stream);

/* Packed sequences (one [1, T, V] row of logits, sequences delimited by cu_seqlens_padded).
 * Replaces from_parallel_logits_to_logprobs_packed_sequences (model_utils.py:1085-1196) at
 * CP = 1: position p of sequence s (start = cu[s], len = cu[s+1]-cu[s]) uses target
 * targets[start + (p+1) % len] unless pre_rolled (then targets[start + p]); the last position of
 * every sequence is dropped; out[s, p] for p < min(len-1, unpacked_seqlen-1), zero elsewhere.
 * logits: [T, vocab] contiguous rows of stride `row_stride`.  cu_seqlens: int32 [n_seq+1] device.
 * out: fp32 [n_seq, unpacked_seqlen-1];  lse_out: fp32 [T] or NULL. */
int nrl_logprob_packed_fwd(const void* logits, int32_t dtype, int64_t total_tokens, int64_t vocab,
                           int64_t row_stride, const int64_t* targets, int32_t pre_rolled,
                           const int32_t* cu_seqlens, int64_t n_seq, int64_t unpacked_seqlen,
                           int64_t vocab_start, int64_t vocab_end, float temperature,
                           int32_t temp_mode, float* out, float* lse_out, void* stream);

/* Backward of the packed entry point: grad is fp32 [n_seq, unpacked_seqlen-1]; dlogits [T, vocab]
 * (rows of stride d_row_stride); dropped / padded positions are zero-filled. */
int nrl_logprob_packed_bwd(const void* logits, int32_t dtype, int64_t total_tokens, int64_t vocab,
                           int64_t row_stride, const int64_t* targets, int32_t pre_rolled,
                           const int32_t* cu_seqlens, int64_t n_seq, int64_t unpacked_seqlen,
                           int64_t vocab_start, int64_t vocab_end, float temperature,
                           int32_t temp_mode, const float* lse, const float* grad, void* dlogits,
                           int64_t d_row_stride, void* stream);

/* ------------------------------------------------------------------------------------------
 * K3  Token logprobs under top-k / top-p filtering.  Replaces apply_top_k_top_p
 * (nemo_rl/algorithms/logits_sampling_utils.py:69-285) followed by log_softmax + gather, i.e.
 * DistributedLogprobWithSampling / ChunkedDistributedLogprobWithSampling at TP = 1
 * (nemo_rl/distributed/model_utils.py:383-719) and the filtered plain branch (:1677-1693), without
 * sorting the vocabulary.  rows->vocab_start must be 0 and vocab_end == vocab.
 * top_k <= 0 and top_p >= 1 switch the respective filter off (at least one must be on).
 * Per row the forward emits the keep predicate (thr_out, tie_out): element v is kept iff
 * x_v > thr, or x_v == thr and v >= tie; and lse_kept_out, the log-sum-exp over the kept set.
 * logprob_out (may be NULL, then rows->targets may be NULL): x_t - lse_kept, or -inf when the target
 * was filtered out.  logprob_unfiltered_out / lse_full_out (may be NULL): the same row's unfiltered
 * logprob (what the KL penalty needs, loss/utils.py:104-118) from the same pass.
 * Rows whose kept set exceeds the on-chip candidate list (4096 entries: a flat distribution under
 * top-p alone, many exact ties, a top_k in the thousands) take a second kernel in the same call that
 * finds the threshold by a radix descent over the logits' order keys instead of sorting (two to four
 * more passes over the row; its sums are integers, so results do not depend on scheduling); there is
 * no limit on top_k or on the kept set.
 * ------------------------------------------------------------------------------------------ */
int nrl_topk_topp_logprob_fwd(const nrl_rows* rows, int64_t top_k, float top_p, float* logprob_out,
                              float* thr_out, int32_t* tie_out, float* lse_kept_out,
                              float* logprob_unfiltered_out, float* lse_full_out, int32_t* kept_count_out,
                              int32_t* kept_index_out, float* kept_value_out, int64_t kept_capacity, void* stream);

/* dlogits_v = keep_v * g * (onehot_v - exp(x_v - lse_kept)); layout arguments as nrl_logprob_bwd.
 * The kept-set record (optional, all of it or none; no counterpart in the reference, which keeps the whole filtered
 * row for autograd): a forward given kept_count_out int32 [rows], kept_index_out int32 [rows, kept_capacity] and
 * kept_value_out fp32 [rows, kept_capacity] (kept_capacity <= 2048) also writes, for every row whose kept set has
 * at most kept_capacity elements, their number, their vocabulary indices and their (temperature-scaled) logits,
 * and -1 as the number for every other row.  A backward given the record back and a dlogits that is one contiguous,
 * 16-byte aligned block (d_stride_inner == vocab, d_stride_outer == d_n_inner * vocab) zero-fills that block and
 * writes only those few entries of a recorded row, without reading the logits; other rows stream as without the
 * record, and so does everything for a strided dlogits.  dlogits may alias the logits (in place, same strides);
 * a dlogits block that overlaps the logits is never cleared first, every row then streams. */
int nrl_topk_topp_logprob_bwd(const nrl_rows* rows, const float* thr, const int32_t* tie,
                              const float* lse_kept, const float* grad, int64_t grad_stride_outer,
                              int64_t grad_stride_inner, const int32_t* kept_count, const int32_t* kept_index,
                              const float* kept_value, int64_t kept_capacity, void* dlogits, int64_t d_n_inner,
                              int64_t d_stride_outer, int64_t d_stride_inner, void* stream);

/* Materialises apply_top_k_top_p's outputs from a forward's (thr, tie): filtered logits (-inf outside
 * the kept set, same dtype, row (o,i) at filtered_out + o*f_stride_outer + i*f_stride_inner) and the
 * keep mask (uint8 [rows, vocab], may be NULL). */
int nrl_topk_topp_filter(const nrl_rows* rows, const float* thr, const int32_t* tie, void* filtered_out,
                         int64_t f_stride_outer, int64_t f_stride_inner, uint8_t* keep_out, void* stream);

/* ------------------------------------------------------------------------------------------
 * K4  ClippedPGLossFn (nemo_rl/algorithms/loss/loss_functions.py:374-788) with calculate_kl and
 * masked_mean (nemo_rl/algorithms/utils.py:42-101, 212-224) fused: loss, its gradient with
 * respect to the token logprobs, and every metric, in two launches.
 * ------------------------------------------------------------------------------------------ */
enum nrl_tis_type { NRL_TIS_NONE = 0, NRL_TIS_TIS = 1, NRL_TIS_ICEPOP = 2, NRL_TIS_SEQ_MASK = 3 };

typedef struct nrl_grpo_cfg {
    int32_t token_level_loss;
    int32_t disable_ppo_ratio;
    int32_t force_on_policy_ratio;
    int32_t use_cispo;
    int32_t sequence_level_importance_ratios;
    int32_t use_importance_sampling_correction;
    int32_t use_on_policy_kl_approximation;
    int32_t tis_type;       /* nrl_tis_type */
    int32_t kl_type;        /* 1, 2, 3 = k1, k2, k3 */
    int32_t has_kl;         /* reference_policy_kl_penalty != 0 */
    int32_t has_kl_input_clamp, has_kl_output_clamp;
    int32_t has_dual_clip;  /* ratio_clip_c is not None */
    int32_t has_nll;        /* positive_example_nll_weight > 0 and "rewards" given */
    float ratio_clip_min, ratio_clip_max, ratio_clip_c;
    float kl_beta, kl_input_clamp, kl_output_clamp;
    float tis_max, tis_min;
    float nll_weight;
} nrl_grpo_cfg;

/* metric slots of the fp32 metrics_out array (NRL_GRPO_N_METRICS entries) */
enum nrl_grpo_metric {
    NRL_M_LOSS = 0, NRL_M_PROBS_RATIO, NRL_M_PROBS_RATIO_CLAMPED, NRL_M_PROBS_RATIO_MIN,
    NRL_M_PROBS_RATIO_MAX, NRL_M_PROBS_RATIO_CLAMPED_MIN, NRL_M_PROBS_RATIO_CLAMPED_MAX,
    NRL_M_KL, /* the reduced kl term (beta included); kl_penalty = this / beta */
    NRL_M_TOKEN_MULT_PROB_ERROR, NRL_M_GEN_KL_ERROR, NRL_M_POLICY_KL_ERROR, NRL_M_JS_DIVERGENCE_ERROR,
    NRL_M_SAMPLING_IMPORTANCE_RATIO, NRL_M_NUM_VALID_SAMPLES, NRL_M_APPROX_ENTROPY, NRL_M_IS_OOB_RATIO,
    NRL_M_POSITIVE_NLL_LOSS, NRL_M_ACTOR_LOSS, NRL_M_N_MASKED_TOKENS, NRL_GRPO_N_METRICS = 24
};

/* Every [B, Sm1] input is fp32 with unit column stride and its own row stride (so the
 * reference's data[...][:, 1:] slices are passed as pointer + 1 with row stride S). */
typedef struct nrl_grpo_inputs {
    int64_t batch, sm1;
    const float* lp;  int64_t lp_stride;   /* current-policy logprobs (requires grad)        */
    const float* lpu; int64_t lpu_stride;  /* unfiltered logprobs for the KL, NULL = use lp  */
    const float* prev; int64_t prev_stride; /* NULL allowed when force_on_policy_ratio        */
    const float* gen; int64_t gen_stride;
    const float* ref; int64_t ref_stride;  /* NULL allowed when !has_kl                      */
    const float* adv; int64_t adv_stride;
    const float* token_mask; int64_t token_mask_stride;
    const float* sample_mask;   /* [B] */
    const float* correct_mask;  /* [B] (rewards > 0), NULL unless has_nll */
    const float* global_valid;  /* device [2]: {global_valid_seqs, global_valid_toks} */
} nrl_grpo_inputs;

int64_t nrl_grpo_loss_workspace_bytes(int64_t batch);

/* loss_out: fp32 [1]; dlp_out: fp32 [B, Sm1] contiguous (d loss / d lp); dlpu_out: fp32 [B, Sm1]
 * or NULL (required iff in->lpu != NULL and cfg->has_kl); metrics_out: fp32 [NRL_GRPO_N_METRICS];
 * workspace: nrl_grpo_loss_workspace_bytes(B) bytes, 8-byte aligned. */
int nrl_grpo_loss_fwd_bwd(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out,
                          float* dlp_out, float* dlpu_out, float* metrics_out, void* workspace,
                          int64_t workspace_bytes, void* stream);

/* nrl_grpo_loss_fwd_bwd without a workspace argument and without any allocation.  It has no counterpart in
 * the reference; it is for callers that cannot allocate device memory around the call: code under HIP graph
 * capture, tight loops, harnesses that forbid hipMalloc.  The per-sequence partial sums live in a fixed
 * array in the library's device image (NRL_GRPO_STATIC_MAX_BATCH * 160 bytes = 1.25 MiB on every GPU the
 * library runs on, held until the process ends); in->batch above NRL_GRPO_STATIC_MAX_BATCH returns
 * NRL_E_WORKSPACE.  Inputs, outputs and results are those of nrl_grpo_loss_fwd_bwd, bit for bit.
 * The first call on a device resolves that device's copy of the array (hipGetSymbolAddress; make it outside a
 * graph capture).  All calls on one GPU share the array: calls that overlap on one GPU (different streams or
 * host threads) race; calls in stream order do not, and nothing needs clearing between them. */
#define NRL_GRPO_STATIC_MAX_BATCH 8192
int nrl_grpo_loss_fwd_bwd_static(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out,
                                 float* dlp_out, float* dlpu_out, float* metrics_out, void* stream);

/* Fused variant: one pass over the logits computes the token logprob (as K1), the loss terms and
 * d loss / d logprob of that token (as K4) and writes dlogits (as K2) from the row held on chip:
 * the logits are read once and the gradient written once.  Replaces, for a single-GPU worker,
 * prepare_loss_input + ClippedPGLossFn + the backward of the logprob op
 * (nemo_rl/algorithms/loss/wrapper.py:292-322 with loss_functions.py:374-788 and
 * nemo_rl/distributed/model_utils.py:120-207).  `in` is as for nrl_grpo_loss_fwd_bwd with lp / lpu
 * ignored (batch = rows->n_outer, sm1 = rows->n_inner).  dlogits holds loss_scale * d loss / d logits
 * (layout as in nrl_logprob_bwd; may alias the logits).  logprob_out: fp32 [B, n_inner]; positions
 * whose mask is zero are not evaluated (logprob 0, zero gradient row, logits not read).
 * Returns NRL_E_UNSUPPORTED for what cannot be fused: sequence-level probability ratios (GSPO), the
 * positive-example NLL term, rows that are not 16-byte aligned or longer than 20480 16-byte vectors.
 * workspace: nrl_fused_workspace_bytes(B, n_inner) bytes, 8-byte aligned. */
int64_t nrl_fused_workspace_bytes(int64_t batch, int64_t n_inner);
int nrl_fused_logits_grpo_loss(const nrl_rows* rows, const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in,
                               float loss_scale, void* dlogits, int64_t d_n_inner, int64_t d_stride_outer,
                               int64_t d_stride_inner, float* logprob_out, float* loss_out,
                               float* metrics_out, void* workspace, int64_t workspace_bytes, void* stream);

/* The same single pass over a packed microbatch: `rows` describes the one packed row (n_outer 1,
 * n_inner = total positions, stride_inner = row stride, targets = packed ids [total] with stride 1),
 * sequence s occupies positions [cu_seqlens[s], cu_seqlens[s+1]) and the loss inputs are [n_seq, in->sm1]
 * with in->sm1 = unpacked_seqlen - 1.  Replaces SequencePackingFusionLossWrapper.__call__ =
 * prepare_packed_loss_input + ClippedPGLossFn + backward (nemo_rl/algorithms/loss/wrapper.py:169-228,
 * loss/utils.py:214-385) at CP = 1.  Position p of a sequence uses target cu[s] + p + 1 (cu[s] + p when
 * the targets are pre-rolled); the last position of every sequence, positions past unpacked_seqlen - 1 and
 * positions outside every sequence get a zero gradient row.  dlogits: [total, vocab] rows of d_row_stride.
 * workspace: nrl_fused_packed_workspace_bytes(n_seq, in->sm1, total) bytes, 8-byte aligned (it also holds one
 * 16-byte record per packed position: where the position sits in the loss inputs). */
int64_t nrl_fused_packed_workspace_bytes(int64_t n_seq, int64_t n_inner, int64_t total);
int nrl_fused_packed_logits_grpo_loss(const nrl_rows* rows, int32_t target_is_pre_rolled, const int32_t* cu_seqlens,
                                      int64_t n_seq, const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in,
                                      float loss_scale, void* dlogits, int64_t d_row_stride, float* logprob_out,
                                      float* loss_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                                      void* stream);

/* NLLLossFn scalar branch (loss_functions.py:818-842): loss = -sum(lp*mask)/(Gt+1e-8);
 * metrics_out[0..2] = {loss, num_unmasked_tokens, num_valid_samples}; dlp_out = -mask/(Gt+1e-8). */
int nrl_nll_loss_fwd_bwd(const nrl_grpo_inputs* in, float* loss_out, float* dlp_out,
                         float* metrics_out, void* workspace, int64_t workspace_bytes, void* stream);

/* calculate_kl (nemo_rl/algorithms/utils.py:42-101) element by element over n fp32 values: logr = reference -
 * logprobs, clamped to +-input_clamp when has_input_clamp; kl_type 1: -logr, 2: logr^2 / 2, 3: exp(logr) - 1 - logr;
 * multiplied by weights[i] when weights is not NULL; clamped to +-output_clamp when has_output_clamp.
 * _bwd writes grad_kl[i] * d kl[i] / d (input) into whichever of the three outputs is not NULL: a token whose logr
 * was clamped passes nothing (neither through the KL nor, as the reference detaches it, through its weight), a
 * value outside the output clamp passes nothing either. */
int nrl_calculate_kl(const float* logprobs, const float* logprobs_reference, const float* weights, int64_t n,
                     int32_t kl_type, int32_t has_input_clamp, float input_clamp, int32_t has_output_clamp,
                     float output_clamp, float* kl_out, void* stream);
int nrl_calculate_kl_bwd(const float* grad_kl, const float* logprobs, const float* logprobs_reference,
                         const float* weights, int64_t n, int32_t kl_type, int32_t has_input_clamp, float input_clamp,
                         int32_t has_output_clamp, float output_clamp, float* dlogprobs_out, float* dreference_out,
                         float* dweights_out, void* stream);

/* masked_mean (nemo_rl/algorithms/utils.py:207-224) over the last axis of fp32 [n_rows, n_cols]:
 * out[r] = sum_c(values * mask) / (norm + 1e-8), norm = sum_c(mask) of the row unless has_norm, then the one value
 * at norm_device (device pointer) or, if that is NULL, norm_host.  The sums are carried in double.  denom_out
 * (or NULL) receives norm + 1e-8 per row for _bwd: dvalues[r, c] = grad_out[r] * mask[r, c] / denom[r]. */
int nrl_masked_mean(const float* values, const float* mask, int64_t n_rows, int64_t n_cols, const float* norm_device,
                    float norm_host, int32_t has_norm, float* out, float* denom_out, void* stream);
int nrl_masked_mean_bwd(const float* grad_out, const float* mask, const float* denom, int64_t n_rows, int64_t n_cols,
                        float* dvalues_out, void* stream);

/* log_softmax over the K logits of a row at the given vocabulary indices (the teacher's top-k), the
 * zero_outside_topk = False branch of get_distillation_topk_logprobs_from_logits
 * (nemo_rl/distributed/model_utils.py:1981-2005): out[r, j] = x[r, idx[r, j]] - logsumexp_j x[r, idx[r, j]].
 * indices: int64 [rows, K] global ids (ids outside [vocab_start, vocab_end) count as -inf), or NULL with
 * K == vocab: plain log_softmax of the row (the teacher's own top-k logits, :2007-2010).  out: fp32 [rows, K].
 * _bwd: dlogits (layout as in nrl_logprob_bwd) is zero except at the K indices, where it holds
 * grad[j] - exp(logprobs[j]) * sum_q grad[q] (summed over duplicates of an index). */
int nrl_topk_logsoftmax_fwd(const nrl_rows* rows, const int64_t* indices, int64_t k, float* out, void* stream);
int nrl_topk_logsoftmax_bwd(const nrl_rows* rows, const int64_t* indices, int64_t k, const float* logprobs,
                            const float* grad, void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner,
                            void* stream);

/* DistillationLossFn (nemo_rl/algorithms/loss/loss_functions.py:1124-1206) on top-k log-probabilities,
 * forward and gradients in one call.  student / teacher logprobs: contiguous fp32 [B, n, K]; h_all: fp32
 * [B, n] (sum_v p log p of the student's full rows) or NULL.  kl_type 0 forward sum t_p (t - s), 1 reverse
 * sum s_p (s - t), 2 mixed with weight mixed_kl_weight on the forward term.  With zero_outside_topk and a
 * non-forward kl_type the correction (H_all - sum s_p s) - log_infinitesimal * (1 - sum s_p) is added (times
 * 1 - mixed_kl_weight when mixed).  With token_mask: loss = sum(per_token * token_mask * sample_mask) /
 * (global_valid_toks[0] + 1e-8); with token_mask == NULL the plain mean over the B * n tokens.
 * d_student_out: fp32 [B, n, K]; d_h_all_out: fp32 [B, n] (written when the correction applies).
 * workspace: nrl_distill_topk_loss_workspace_bytes(B, n) bytes, 8-byte aligned. */
int64_t nrl_distill_topk_loss_workspace_bytes(int64_t batch, int64_t n);
int nrl_distill_topk_loss_fwd_bwd(const float* student_logprobs, const float* teacher_logprobs, const float* h_all,
                                  const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                                  const float* global_valid_toks, int64_t batch, int64_t n, int64_t k,
                                  int32_t kl_type, float mixed_kl_weight, int32_t zero_outside_topk,
                                  float log_infinitesimal, float* loss_out, float* d_student_out, float* d_h_all_out,
                                  void* workspace, int64_t workspace_bytes, void* stream);

/* NLLLossFn per-sample branch (dpo_loss=True, loss_functions.py:823-829): loss_rows_out[b] =
 * -sum_t lp[b,t] * token_mask[b,t] * sample_mask[b], divided by max(sum_t mask, 1) with
 * average_log_probs; den_out[b] is that divisor (1 without averaging); totals_out[0..1] =
 * {num_unmasked_tokens, num_valid_samples}.  workspace: B floats.  _bwd: dlp_out[b,t] =
 * -token_mask * sample_mask[b] / den[b] * grad_rows[b], contiguous [B, n]. */
int nrl_nll_rows_fwd(const float* lp, int64_t lp_stride, const float* token_mask, int64_t token_mask_stride,
                     const float* sample_mask, int64_t batch, int64_t n, int32_t average_log_probs,
                     float* loss_rows_out, float* den_out, float* totals_out, void* workspace,
                     int64_t workspace_bytes, void* stream);
int nrl_nll_rows_bwd(const float* grad_rows, const float* token_mask, int64_t token_mask_stride,
                     const float* sample_mask, const float* den, int64_t batch, int64_t n, float* dlp_out,
                     void* stream);

/* DPOLossFn (loss_functions.py:1025-1106) on token logprobs, forward and gradient in one call.  Rows
 * alternate chosen / rejected (batch must be even).  reward[b] = sum_t (lp - ref) * token_mask (/ max(sum_t
 * token_mask, 1) with preference_average_log_probs); preference = sum_p -logsigmoid(beta * (reward_c -
 * reward_r)) * sample_mask_c^2 / (Gs/2 + 1e-8) with Gs = global_valid[0]; the SFT term (weight > 0) is the
 * chosen rows' per-sample NLL, masked-mean over the pairs in the same way.  ref may be NULL (zeros); the
 * caller passes it already aligned with lp (the reference reads reference_policy_logprobs[:, :-1]).
 * metrics_out[0..6] = {loss, sft_loss, preference_loss, accuracy, rewards_chosen_mean,
 * rewards_rejected_mean, num_valid_samples}; dlp_out: contiguous fp32 [B, n].
 * workspace: nrl_dpo_workspace_bytes(B) bytes. */
int64_t nrl_dpo_workspace_bytes(int64_t batch);
int nrl_dpo_loss_fwd_bwd(const float* lp, int64_t lp_stride, const float* ref, int64_t ref_stride,
                         const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                         const float* global_valid, int64_t batch, int64_t n, float beta,
                         float preference_loss_weight, float sft_loss_weight,
                         int32_t preference_average_log_probs, int32_t sft_average_log_probs, float* loss_out,
                         float* dlp_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                         void* stream);

/* PreferenceLossFn (loss_functions.py:877-946): rewards [B] from a reward model, beta = 1.
 * metrics_out[0..4] = {loss, accuracy, rewards_chosen_mean, rewards_rejected_mean, num_valid_samples};
 * drewards_out: fp32 [B]. */
int nrl_preference_loss_fwd_bwd(const float* rewards, const float* sample_mask, const float* global_valid,
                                int64_t batch, float* loss_out, float* drewards_out, float* metrics_out,
                                void* stream);

/* ------------------------------------------------------------------------------------------
 * K5  calculate_baseline_and_std_per_prompt (nemo_rl/algorithms/utils.py:104-198) and
 * GRPOAdvantageEstimator.compute_advantage (nemo_rl/algorithms/advantage_estimator.py:82-98).
 * prompts: int64 [B, Sp] rows of stride prompt_stride; rows are grouped by exact equality.
 * group_out (int32 [B], may be NULL): index of the first row of each row's group.
 * std_rewards may be NULL (= rewards).  adv_out (fp32 [B]) may be NULL; when given it holds
 * (r - baseline), divided by (std + 1e-6) where std > 0 if `normalize`.
 * workspace: nrl_group_workspace_bytes(B) bytes.
 * ------------------------------------------------------------------------------------------ */
int64_t nrl_group_workspace_bytes(int64_t batch);
int nrl_group_baseline_std(const int64_t* prompts, int64_t batch, int64_t prompt_len,
                           int64_t prompt_stride, const float* rewards, const float* valid,
                           const float* std_rewards, int32_t leave_one_out, int32_t normalize,
                           float* baseline_out, float* std_out, float* adv_out, int32_t* group_out,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Full-vocabulary reductions of the distillation losses, on the K1 / K2 streaming core (TP = 1).
 * `rows` describes the logits as for nrl_logprob_fwd; its `targets` / temperature fields are not used.
 * Gradients are written in the logits' dtype (one narrowing of the fp32 value); dlogits must not alias
 * the logits.
 *
 * nrl_neg_entropy_*: ChunkedDistributedEntropy (nemo_rl/distributed/model_utils.py:2023-2103):
 *   h_out[r] = sum_v p_v log p_v, lse_out[r]; backward g * p_v * (log p_v - h).
 * nrl_gather_logprob_*: ChunkedDistributedGatherLogprob (model_utils.py:722-836): out[r, k] = log p at
 *   indices[r, k] (int64 [rows, K], global ids; 0 outside [vocab_start, vocab_end)); backward
 *   -p_v * sum_k g_k + sum over the k with indices[r, k] == v of g_k.
 * nrl_soft_cross_entropy_*: DistributedCrossEntropy (model_utils.py:209-264): ce_out[r] =
 *   -sum_v softmax(teacher)_v * log_softmax(student)_v; backward g * (softmax(student) - softmax(teacher)).
 *   teacher: same dtype and [n_outer, n_inner, vocab] shape as the student, with its own row strides.
 * ------------------------------------------------------------------------------------------ */
int nrl_neg_entropy_fwd(const nrl_rows* rows, float* h_out, float* lse_out, void* stream);
int nrl_neg_entropy_bwd(const nrl_rows* rows, const float* lse, const float* h, const float* grad, void* dlogits,
                        int64_t d_stride_outer, int64_t d_stride_inner, void* stream);
int nrl_gather_logprob_fwd(const nrl_rows* rows, const int64_t* indices, int64_t k, float* out, float* lse_out,
                           void* stream);
int nrl_gather_logprob_bwd(const nrl_rows* rows, const int64_t* indices, int64_t k, const float* lse, const float* grad,
                           void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner, void* stream);
int nrl_soft_cross_entropy_fwd(const nrl_rows* student, const void* teacher, int64_t t_stride_outer,
                               int64_t t_stride_inner, float* ce_out, float* lse_student_out, float* lse_teacher_out,
                               void* stream);
int nrl_soft_cross_entropy_bwd(const nrl_rows* student, const void* teacher, int64_t t_stride_outer,
                               int64_t t_stride_inner, const float* lse_student, const float* lse_teacher,
                               const float* grad, void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner,
                               void* stream);

/* Ascending indices of the non-zero entries of values [n] (NaN counts as non-zero) and their number: the
 * selection `arange(n)[std != 0.0]` of dynamic_sampling (nemo_rl/algorithms/grpo.py:1752-1758).
 * indices_out: int32 [n] (the first *count_out entries are written). */
int nrl_nonzero_indices(const float* values, int64_t n, int32_t* indices_out, int32_t* count_out, void* stream);

/* Per-sequence multiplicative logprob error and the mask that drops sequences above a threshold.
 * Replaces compute_and_apply_seq_logprob_error_masking (nemo_rl/algorithms/grpo.py:2513-2640):
 * err[b] = sum_t exp(|gen - prev| * m) * m / max(sum_t m, 1) over t >= 1 with m = token_mask[b,t] * sample_mask[b]
 * (0 for a sequence without unmasked tokens); with a threshold sample_mask_out[b] = (err[b] <= threshold) *
 * sample_mask[b], otherwise a copy of sample_mask.
 * All tensors fp32; prev / gen / token_mask [B, S] with their row strides; rewards [B] or NULL.
 * record_out (fp32 [8]): max, mean, min error over sequences with unmasked tokens; the same three over the
 * sequences that stay; number of newly masked sequences; fraction of those with reward == 1.
 * workspace: B floats. */
int nrl_seq_logprob_error(const float* prev, int64_t prev_stride, const float* gen, int64_t gen_stride,
                          const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                          const float* rewards, int64_t batch, int64_t seq_len, int32_t has_threshold,
                          float threshold, float* seq_err_out, float* sample_mask_out, float* record_out,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * K6  Fused lm_head -> token logprob on the bf16 matrix cores (MFMA), without a pass over [N, V]
 * logits in fp32.  Replaces ChunkedDistributedHiddenStatesToLogprobs
 * (nemo_rl/distributed/model_utils.py:2137-2316) at TP = 1.
 * hidden: bf16 [N, H] rows of stride ldh (token order is the caller's); weight: bf16 [V, H] rows of
 * stride ldw; both 16-byte aligned, H and the strides multiples of 8.  targets: int64 [N], already
 * shifted.  The logits of a tile are rounded to bf16 before the softmax, as the reference's bf16
 * matmul does.  logprob_out / lse_out: fp32 [N] (lse_out may be NULL).
 * Backward: grad fp32 [N] -> dhidden_out fp32 [N, H] (row stride ld_dh) and dweight_out bf16 [V, H]
 * (row stride ld_dw), accumulated in fp32 and narrowed once.  Tokens are processed in chunks of 16384:
 * per chunk the gradient of the logits exists as bf16 [chunk, V] (twice, one transposed).
 * Kept logits (a choice of the caller, who has the memory or not): with logits_out not NULL the forward
 * also writes the bf16 logits into that buffer (16-byte aligned, nrl_lmhead_kept_logits_bytes(N, V) bytes:
 * 2 bytes per token and id, both rounded up to multiples of 32); handed back as logits_kept the backward reads
 * them instead of multiplying hidden and weight a second time (the reference always recomputes, :2249-2262,
 * because its logits are fp32 and its memory a quarter).  Both ways give the same gradients: the kept values are
 * the rounded logits the recomputation arrives at.  The buffer is for the backward only; its layout is the one
 * the matrix instructions leave in registers: blocks of 32 ids x 32 tokens, 2 KiB each, ceil(V / 32) blocks per
 * token block; inside a block [half p = 0, 1][lane = 32 h + token % 32][8 values], the 8 values being the ids
 * 16 p + 8 q + 4 h + e of the block (q = 0, 1; e = 0..3).  Ids and tokens past the end hold unspecified values.
 * Workspaces: nrl_lmhead_*_workspace_bytes(), 256-byte aligned.
 * Environment (read once per process): NRL_LMHEAD_ALIGN -- the forward's workgroups that share an L2 wait for
 * each other before their first tile (unset), before every N-th tile (N > 0), or never (0);
 * NRL_LMHEAD_ALIGN_SPINS -- polls after which a workgroup stops waiting (default 512; the wait is always
 * bounded).  The results are the same whatever they say.
 * ------------------------------------------------------------------------------------------ */
int64_t nrl_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t vocab);
int64_t nrl_lmhead_kept_logits_bytes(int64_t n_tokens, int64_t vocab);
int nrl_lmhead_logprob_fwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                           const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                           int64_t vocab_start, int64_t vocab_end, float* logprob_out, float* lse_out,
                           void* logits_out, int64_t logits_bytes, void* workspace, int64_t workspace_bytes,
                           void* stream);
int64_t nrl_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab);
int nrl_lmhead_logprob_bwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                           const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                           int64_t vocab_start, int64_t vocab_end, const float* lse, const float* grad,
                           const void* logits_kept, int64_t logits_bytes, float* dhidden_out, int64_t ld_dh,
                           void* dweight_out, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                           void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NRL_HIP_H */
