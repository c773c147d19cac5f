/*
 * openrlhf_amd.h — C ABI of libopenrlhf_amd.so: hand-written gfx950 (MI355X) kernels for the
 * token-level RL numerics of OpenRLHF.
 *
 * The reference has no FFI layer for this path: its boundary is the Python signature of a set of
 * torch functions. Each entry point below replaces the device work of one of them and cites it
 * as `file:line` relative to the OpenRLHF source tree. A Python binding (ctypes) passes
 * `tensor.data_ptr()`, element counts and the HIP stream; nothing here knows about torch.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless the comment says "host";
 *  - every function returns ORLHF_OK (0) or a negative error code, never throws, and leaves a
 *    thread-local message readable with orlhf_last_error();
 *  - kernels are launched asynchronously on `stream` (a hipStream_t; NULL = default stream) and
 *    the call does not synchronise; the library keeps no device state between calls and
 *    allocates no device memory: outputs, saved row statistics and workspaces are the caller's;
 *  - per-token tensors come in one of two row layouts, selected by `cu_seqlens`:
 *      padded : cu_seqlens == NULL, contiguous [n_rows, n_cols]; row b token t at b*n_cols + t;
 *      packed : cu_seqlens != NULL, int64 [n_rows + 1] on the device; row b holds tokens
 *               cu_seqlens[b] .. cu_seqlens[b+1]-1 of one flat array and n_cols is an upper
 *               bound of the longest row (it only sizes the launch);
 *  - masks are read as float weights (the reference multiplies by the mask): ORLHF_MASK_U8 for
 *    torch.bool / torch.uint8, ORLHF_MASK_F32, ORLHF_MASK_I64, or ORLHF_MASK_NONE (all ones,
 *    pointer ignored);
 *  - reductions are two-stage and deterministic (no floating-point atomics): the same inputs give
 *    the same bits on every run.
 */
#ifndef OPENRLHF_AMD_H
#define OPENRLHF_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORLHF_ABI_VERSION 23

#define ORLHF_OK 0
#define ORLHF_ERR_INVALID_ARG (-1) /* null pointer, bad size / dtype / enum                     */
#define ORLHF_ERR_LAUNCH (-2)      /* hipGetLastError() after a launch reported a failure       */
#define ORLHF_ERR_UNSUPPORTED (-3) /* a combination the kernels do not implement                */

enum orlhf_dtype { ORLHF_F32 = 0, ORLHF_BF16 = 1, ORLHF_F16 = 2 };
enum orlhf_mask_dtype { ORLHF_MASK_NONE = 0, ORLHF_MASK_U8 = 1, ORLHF_MASK_F32 = 2, ORLHF_MASK_I64 = 3 };
enum orlhf_kl_estimator { ORLHF_KL_K1 = 0, ORLHF_KL_K2 = 1, ORLHF_KL_K3 = 2 };
enum orlhf_agg_mode {
  ORLHF_AGG_TOKEN_MEAN = 0, /* sum(x*m) / (sum(m) | batch_num_tokens) * dp_size                  */
  ORLHF_AGG_SEQ_MEAN = 1,   /* mean over non-empty rows of sum(x*m)/(sum(m)+1e-8)               */
  ORLHF_AGG_ROW_MEAN = 2,   /* per-row sum(x*m)/sum(m), output [n_rows] (masked_mean, dim=-1)   */
  ORLHF_AGG_SEQ_MEAN_TOKEN_SUM = 3 /* mean over non-empty rows of sum(x*m): not in the reference  */
};
enum orlhf_policy_type { ORLHF_POLICY_PPO = 0, ORLHF_POLICY_GSPO = 1 };
enum orlhf_is_correction { ORLHF_IS_NONE = 0, ORLHF_IS_TIS = 1, ORLHF_IS_ICEPOP = 2, ORLHF_IS_SEQ_MASK_TIS = 3 };
enum orlhf_pair_loss {
  ORLHF_PAIR_DPO_SIGMOID = 0, /* DPOLoss, ipo=False (label smoothing = conservative DPO)   */
  ORLHF_PAIR_DPO_IPO = 1,     /* DPOLoss, ipo=True                                          */
  ORLHF_PAIR_LOGSIGMOID = 2,  /* PairWiseLoss: -logsigmoid(chosen - rejected [- margin])    */
  ORLHF_PAIR_LOGEXP = 3       /* LogExpLoss: log(1 + exp(rejected - chosen))                */
};
enum orlhf_group_estimator {
  ORLHF_GROUP_IDENTITY = 0, /* gae, reinforce: rewards unchanged                                 */
  ORLHF_GROUP_RLOO = 1,     /* r - (sum - r)/(n-1)                                               */
  ORLHF_GROUP_BASELINE = 2, /* reinforce_baseline, dr_grpo: r - mean                             */
  ORLHF_GROUP_NORM = 3      /* group_norm: (r - mean)/(std_unbiased + 1e-9)                      */
};

typedef void* orlhf_stream_t; /* hipStream_t */

/* Library ABI version (ORLHF_ABI_VERSION of the build). No reference counterpart. */
int orlhf_version(void);
/* Message of the last failing call on this host thread ("" if none). No reference counterpart. */
const char* orlhf_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Vocabulary-row kernels
 * ---------------------------------------------------------------------------------------- */

/* `flags` of orlhf_logprob_entropy_fwd: reserved, must be 0. */

/*
 * Fused log-softmax + gather + entropy over full vocabulary rows, one streaming pass.
 *   logprob[i] = z[i,label_i] - logsumexp_j z[i,j],  z = logits / temperature
 *   entropy[i] = logsumexp_j x[i,j] - sum_j softmax(x)[i,j] * x[i,j],  x = logits (unscaled)
 * Replaces log_probs_from_logits (openrlhf/models/utils.py:139-163, incl. _logsumexp_by_chunk
 * :129-136 and the flash-attn cross_entropy_loss call :147-150) and compute_entropy
 * (openrlhf/models/utils.py:182-186) as called from Actor.forward
 * (openrlhf/models/actor.py:265-296: entropy before the temperature division, log-prob after).
 *   logits    [n_rows, vocab], element stride 1, `row_stride` elements between rows
 *   labels    int64 [n_rows]; label -100 gives logprob 0 (flash-attn ignore_index), any other
 *             label outside [0, vocab) gives NaN; neither reads out of bounds
 *   logprob   float [n_rows] or NULL;  entropy float [n_rows] or NULL (not both NULL)
 *   row_stats float [n_rows, 4] or NULL: {lse(z), lse(x), E_softmax(x)[x], 0}, what the backward
 *             needs; fp32 accumulation and fp32 outputs for every input dtype
 *   row_mask  uint8 [n_rows] or NULL: rows with 0 are not read; their outputs and statistics are
 *             0. This is how the caller skips prompt and padding positions, whose log-probs
 *             Actor.forward multiplies by 0 anyway (openrlhf/models/actor.py:294).
 */
int orlhf_logprob_entropy_fwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                              int64_t row_stride, const int64_t* labels, double temperature,
                              float* logprob, float* entropy, float* row_stats,
                              const uint8_t* row_mask, int flags, orlhf_stream_t stream);

/*
 * logits[i,j] <- logits[i,j] / divisor, rounded to `dtype`, in place: the side effect of
 * logits.div_(temperature) in log_probs_from_logits (openrlhf/models/utils.py:140-141), for
 * callers that read the scaled logits afterwards. The log-prob entry points never need it (they
 * fold the division into their loads).
 */
int orlhf_divide_rows_inplace(void* logits, int dtype, int64_t n_rows, int64_t vocab,
                              int64_t row_stride, double divisor, orlhf_stream_t stream);

/*
 * The same forward for launches with fewer rows than the GPU has compute units (short rollouts,
 * a 64-token micro-batch): every row is cut into segments, one workgroup per (row, segment)
 * writes a partial record (running maxima and sums) into `workspace`, and the records of a row are
 * merged in segment order, in fp64, and the row finished as the whole-row kernel does. Same
 * arguments, outputs and conventions as orlhf_logprob_entropy_fwd (same reference lines:
 * openrlhf/models/utils.py:139-163,182-186); results agree with it to the rounding of the fp32
 * partial sums. orlhf_logprob_entropy_split_workspace_bytes returns the bytes this shape needs, 0
 * when the rows would not be cut (256 rows or more, or rows shorter than 64 KiB); then the call is
 * orlhf_logprob_entropy_fwd itself and `workspace` may be NULL. The cut depends on the shape
 * only. orlhf_logprob_entropy_bwd needs no workspace and cuts its rows by the same rule itself.
 *
 * Who merges: with `tickets` NULL a second small kernel does. With `tickets` (n_rows int32, ALL
 * ZERO on entry) the forward kernel does it itself: every segment draws a ticket of its row when
 * its record is written, and the workgroup that draws the last one merges the row and puts the
 * ticket back to zero, so one launch is all and the same array serves the next call unchanged.
 * Nothing waits for anything. Both ways merge the same records in the same order: the outputs are
 * bit-identical. Calls that may overlap on the GPU need ticket arrays of their own, and an array
 * whose call was aborted midway has to be zeroed again.
 */
int64_t orlhf_logprob_entropy_split_workspace_bytes(int dtype, int64_t n_rows, int64_t vocab);
int orlhf_logprob_entropy_fwd_split(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                    int64_t row_stride, const int64_t* labels, double temperature,
                                    float* logprob, float* entropy, float* row_stats,
                                    const uint8_t* row_mask, void* workspace, int64_t workspace_bytes,
                                    int32_t* tickets, orlhf_stream_t stream);

/*
 * Backward of the above in one streaming pass, written in the logits dtype:
 *   grad[i,j] = g_logprob[i] * (1[j==label_i] - softmax(z)[i,j]) / temperature
 *             + g_entropy[i] * softmax(x)[i,j] * (E[x] - x[i,j])
 * `grad_logits` may alias `logits` (in-place: each 16-byte chunk is read, then overwritten by the
 * same lane). Replaces torch autograd through openrlhf/models/utils.py:139-163 and :182-186.
 * g_logprob / g_entropy: float [n_rows] or NULL (treated as 0). Rows whose upstream gradients
 * are both exactly 0, and rows with row_mask 0 (same array as in the forward, or NULL), are
 * written as zeros without reading their logits.
 */
int orlhf_logprob_entropy_bwd(const void* logits, void* grad_logits, int dtype, int64_t n_rows,
                              int64_t vocab, int64_t row_stride, int64_t grad_row_stride,
                              const int64_t* labels, double temperature, const float* g_logprob,
                              const float* g_entropy, const float* row_stats,
                              const uint8_t* row_mask, orlhf_stream_t stream);

/*
 * Forward and backward in ONE pass for callers that know the upstream weights when the forward
 * runs, i.e. whose loss is sum_i w_logprob[i]*logprob[i] + w_entropy[i]*entropy[i] (SFT:
 * w_logprob = -mask/N, openrlhf/models/loss.py:104): computes logprob / entropy exactly as
 * orlhf_logprob_entropy_fwd and writes d(loss)/d(logits) exactly as orlhf_logprob_entropy_bwd
 * with g = w, but reads every logits row once (the row stays in the registers of one CU), so a
 * token costs 2*V*sizeof(dtype) bytes of HBM traffic instead of 3*V*sizeof(dtype). Rows longer
 * than the registers hold (155648 bf16/fp16 or 77824 fp32 elements) keep their first 131072 /
 * 65536 elements there and stream the rest twice (2.5*V at V = 262144).
 * Replaces the same reference lines as the two calls above (openrlhf/models/utils.py:129-163,
 * 182-186 and their autograd). grad_logits may alias logits. w_* / logprob / entropy nullable
 * (a NULL weight array is all zeros). Returns ORLHF_ERR_UNSUPPORTED when a row is too long for
 * that to pay (vocab > orlhf_logprob_entropy_fwd_bwd_max_vocab(dtype): 524288 for bf16/fp16,
 * 262144 for fp32) or when logits and grad rows differ in their 16-byte phase; callers then use
 * the two separate entry points.
 */
int64_t orlhf_logprob_entropy_fwd_bwd_max_vocab(int dtype);
int orlhf_logprob_entropy_fwd_bwd(const void* logits, void* grad_logits, int dtype, int64_t n_rows,
                                  int64_t vocab, int64_t row_stride, int64_t grad_row_stride,
                                  const int64_t* labels, double temperature, const float* w_logprob,
                                  const float* w_entropy, float* logprob, float* entropy,
                                  const uint8_t* row_mask, orlhf_stream_t stream);

/*
 * lm-head + log-prob + entropy without the [n_rows, vocab] logits (or with as much of them as the
 * caller has room for): what Actor.forward does between the last hidden states and the action
 * log-probs (openrlhf/models/actor.py:263-285: the model's lm_head projection,
 * output["logits"].to(float32), compute_entropy, log_probs_from_logits) as matrix-core tiles whose
 * logits are folded into per-token statistics in registers.
 *   logits[i, v] = round_to_dtype(sum_h hidden[i, h] * weight[v, h])   (fp32 accumulation; the 16-bit
 *                  rounding is the one the reference's lm_head output has before its fp32 up-cast)
 *   logprob / entropy / row_stats as orlhf_logprob_entropy_fwd on those logits
 *   hidden  [n_rows, hidden_dim] and weight [vocab, hidden_dim] (the nn.Linear layout), bf16 or
 *           fp16 (`dtype`), element stride 1, row strides in elements below 2^23; both 4-byte
 *           aligned with even strides and an even hidden_dim (else ORLHF_ERR_UNSUPPORTED)
 *   labels  int64 [n_rows] (-100: logprob 0; any other label outside [0, vocab): NaN)
 *   kept_logits [n_rows, kept_stride] of `dtype`, or NULL with kept_cols = 0: the logits of the
 *           first kept_cols vocabulary columns are stored there (the tiles produce them anyway), so
 *           that the backward need not recompute them. kept_cols is a multiple of 256, at most the
 *           vocabulary rounded up to 256 (then all logits are kept; columns past the vocabulary hold
 *           a large negative filler, which the backward overwrites with zeros); kept_stride >= kept_cols, a multiple of 8; 16-byte aligned. Results do not
 *           depend on kept_cols.
 *   workspace: orlhf_lmhead_workspace_bytes(n_rows, hidden_dim, vocab, kept_cols, 0) bytes, 256-byte aligned
 */
int64_t orlhf_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab, int64_t kept_cols,
                                     int backward);
int orlhf_lmhead_logprob_entropy_fwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                     int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                     int64_t weight_stride, const int64_t* labels, double temperature,
                                     float* logprob, float* entropy, float* row_stats, void* kept_logits,
                                     int64_t kept_cols, int64_t kept_stride, void* workspace,
                                     int64_t workspace_bytes, orlhf_stream_t stream);
/*
 * Backward of the above down to the hidden states and the lm_head weight (torch autograd through
 * openrlhf/models/actor.py:263-285 and the projection): with P = d(loss)/d(logits) as in
 * orlhf_logprob_entropy_bwd, rounded to `dtype` (the dtype the reference's logits gradient has),
 *   grad_hidden[i, h] = sum_v P[i, v] * weight[v, h]         grad_weight[v, h] = sum_i P[i, v] * hidden[i, h]
 * both accumulated in fp32 and rounded once to `dtype`. Over the kept columns P is written OVER
 * kept_logits (the logits are gone afterwards); the rest of the vocabulary is processed in chunks:
 * per chunk the logits tiles are recomputed, P is written to the workspace and multiplied twice on
 * the matrix cores. The gradients are the same bits for every kept_cols and every chunk width (the
 * kept logits are what the recompute rounds to, and grad_hidden's sum over the vocabulary is
 * continued in the accumulators in one fixed order). kept_logits / kept_cols / kept_stride: as
 * passed to the forward of the same inputs. grad_hidden [n_rows, hidden_dim] / grad_weight
 * [vocab, hidden_dim]: either may be NULL; row strides in elements. row_stats: from the forward.
 * Rows whose upstream gradients are both 0 contribute exact zeros.
 *   workspace: orlhf_lmhead_workspace_bytes(n_rows, hidden_dim, vocab, kept_cols, 1) bytes or more
 *   (a larger workspace means wider chunks), 256-byte aligned.
 */
int orlhf_lmhead_logprob_entropy_bwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                     int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                     int64_t weight_stride, const int64_t* labels, double temperature,
                                     const float* g_logprob, const float* g_entropy,
                                     const float* row_stats, void* kept_logits, int64_t kept_cols,
                                     int64_t kept_stride, void* grad_hidden, int64_t grad_hidden_stride,
                                     void* grad_weight, int64_t grad_weight_stride, void* workspace,
                                     int64_t workspace_bytes, orlhf_stream_t stream);

/*
 * The loss assembly of the PPO actor step (openrlhf/trainer/ray/ppo_actor.py:305-352) folded into
 * the one-pass kernel: for every logits row the kernel computes logprob and entropy, evaluates
 *   loss = sum_i policy_coef[i] * L_ppo(lp_i; old_i, adv_i [, rollout_i])       (loss.py:166-218)
 *        + kl_coef * sum_i token_coef[i] * KL_est(lp_i - base_i)                (utils.py:78-95)
 *        - entropy_coef * sum_i token_coef[i] * entropy_i
 * 's derivative wrt logprob_i and entropy_i on the spot, and writes d(loss)/d(logits), all with
 * one read and one write of the logits. All arrays are float [n_rows], aligned with the logits
 * rows. policy_coef / token_coef are the aggregation weights (row_coef of
 * orlhf_masked_aggregate_fwd times the mask, times any loss scale); rows where both are 0 get a
 * zero gradient. Token-level importance corrections only (TIS, ICEPOP); GSPO and seq-mask-TIS need
 * a sequence-level ratio before any token can be differentiated and are not fusable. The loss
 * VALUES are obtained afterwards from the returned per-token logprob / entropy with
 * orlhf_policy_loss_fwd, orlhf_approx_kl_fwd and orlhf_masked_aggregate_fwd (17 B/token).
 */
typedef struct orlhf_step_terms {
  const float* old_log_probs;
  const float* advantages;
  const float* rollout_log_probs; /* NULL unless is_correction != NONE */
  const float* base_log_probs;    /* NULL: no KL term */
  const float* policy_coef;
  const float* token_coef;
  float clip_eps_low, clip_eps_high;
  float dual_clip;                /* <= 0: off */
  int is_correction;              /* ORLHF_IS_NONE / _TIS / _ICEPOP */
  float is_low, is_high;
  int kl_estimator;               /* orlhf_kl_estimator */
  float kl_coef;
  float entropy_coef;
} orlhf_step_terms;

int orlhf_policy_step_fwd_bwd(const void* logits, void* grad_logits, int dtype, int64_t n_rows,
                              int64_t vocab, int64_t row_stride, int64_t grad_row_stride,
                              const int64_t* labels, double temperature, const orlhf_step_terms* terms,
                              float* logprob, float* entropy, const uint8_t* row_mask,
                              orlhf_stream_t stream);

/*
 * Index work around orlhf_policy_step_fwd_bwd, one launch instead of a dozen framework launches.
 * The per-token terms of the actor step live in [B, A] tensors (the last A of the first T-1
 * columns of a padded [B, T] batch, openrlhf/models/actor.py:287-296); the vocabulary-row kernel
 * wants one value per logits row: row r is flat position packed_indices[r] (or r when
 * packed_indices is NULL and n_rows = B*T) of the [B, T] grid, i.e. (b, t) with action column
 * t - (T - 1 - A). For every row this writes
 *   labels_rows      sequences[b, (t + 1) mod T]  (torch.roll(sequences, -1, 1): actor.py:273-276)
 *   weight_rows      action_mask[b, col] as a float, 0 outside the action columns; need_rows = (weight != 0)
 *   old / adv / rollout / base rows: the [B, A] value at (b, col), 0 outside the action columns
 *   policy_coef_rows = row_coef_policy[b] * weight * loss_scale, token_coef_rows likewise with
 *                      row_coef_token (row_coef of orlhf_masked_aggregate_fwd: the weight of a
 *                      token in aggregate_loss, openrlhf/models/loss.py:11-39)
 * rollout / base inputs and outputs are nullable together. Replaces the slicing / masking /
 * re-padding index arithmetic of openrlhf/models/actor.py:273-296 and
 * openrlhf/models/ring_attn_utils.py:129-140,181 for the fused step.
 */
int orlhf_actor_step_gather(const int64_t* sequences, const void* action_mask, int mask_dtype,
                            const int64_t* packed_indices, int64_t batch, int64_t seqlen, int64_t width,
                            int64_t n_rows, const float* old_log_probs, const float* advantages,
                            const float* rollout_log_probs, const float* base_log_probs,
                            const float* row_coef_policy, const float* row_coef_token, float loss_scale,
                            int64_t* labels_rows, uint8_t* need_rows, float* weight_rows, float* old_rows,
                            float* adv_rows, float* rollout_rows, float* base_rows,
                            float* policy_coef_rows, float* token_coef_rows, orlhf_stream_t stream);
/*
 * Every value the actor training step reports (openrlhf/trainer/ray/ppo_actor.py:305-352), from the
 * per-row log-probs / entropies orlhf_policy_step_fwd_bwd returned and the per-row arrays above,
 * in two launches (deterministic two-stage fp64 sums), plus the scatter of the per-row results
 * back to [B, A]:
 *   out8 = { loss, actor_loss, clip_ratio, ppo_kl, vllm_kl, kl_loss, entropy_loss, logprobs_diff }
 *   loss = actor_loss + kl_coef * kl_loss - entropy_coef * entropy_loss (the last only if
 *   entropy_in_loss); vllm_kl / kl_loss / logprobs_diff / entropy_loss are NaN when their inputs
 *   (rollout_rows / base_rows / entropy_rows) are NULL.
 *   action_log_probs [B, A] <- logprob * weight and action_entropy [B, A] <- entropy at the rows'
 *   action columns; positions no row maps to are left untouched (the caller zero-fills).
 * Since policy_coef / token_coef are exactly d(aggregate_loss)/d(token loss) (times loss_scale),
 * the aggregated losses are their dot products with the token losses.
 * workspace: orlhf_actor_step_values_workspace_bytes(n_rows) bytes.
 */
int64_t orlhf_actor_step_values_workspace_bytes(int64_t n_rows);
int orlhf_actor_step_values(const float* logprob_rows, const float* entropy_rows, const float* weight_rows,
                            const float* old_rows, const float* adv_rows, const float* rollout_rows,
                            const float* base_rows, const float* policy_coef_rows,
                            const float* token_coef_rows, const int64_t* packed_indices, int64_t seqlen,
                            int64_t width, int64_t n_rows, const orlhf_step_terms* terms, float loss_scale,
                            int entropy_in_loss, void* workspace, float* action_log_probs,
                            float* action_entropy, float* out8, orlhf_stream_t stream);

/*
 * data[i] *= g[0] / expected, skipped entirely (every workgroup returns at once) when the ratio
 * is 1: lets an autograd backward hand out a gradient that was produced ahead of time with the
 * scale `expected` and still be correct if the upstream gradient turns out different, without a
 * host synchronisation. No reference counterpart.
 */
int orlhf_rescale_inplace_if(void* data, int dtype, int64_t n, const float* g, float expected,
                             orlhf_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Per-token kernels: KL, masked aggregation, PPO policy loss, value loss
 * ---------------------------------------------------------------------------------------- */

/*
 * out = clamp(k(lp - base), -10, 10); k1: d, k2: d*d/2, k3: exp(-d) - 1 + d; fp32 out.
 * Replaces compute_approx_kl (openrlhf/models/utils.py:64-95). `dtype` is the type of both
 * inputs (the reference up-casts with .float()). n = number of elements (flat).
 */
int orlhf_approx_kl_fwd(const void* log_probs, const void* log_probs_base, int dtype, int64_t n,
                        int estimator, float* out, orlhf_stream_t stream);
/* g_lp = g_out * d(out)/d(lp) (0 where the clamp is active, closed interval passes);
 * g_base (nullable) = -g_lp. Autograd of openrlhf/models/utils.py:78-95. */
int orlhf_approx_kl_bwd(const void* log_probs, const void* log_probs_base, int dtype, int64_t n,
                        int estimator, const float* g_out, float* g_lp, float* g_base,
                        orlhf_stream_t stream);

/* Normaliser of a token/sequence aggregate (openrlhf/models/loss.py:29-39,
 * openrlhf/utils/loss_utils.py:15-105). norm_dev != NULL: read the denominator from that device
 * float; else norm_value if it is not NaN; else the local sum over the mask (token mode) or the
 * local count of non-empty rows (sequence mode). */
typedef struct orlhf_norm {
  double dp_size;
  double norm_value;     /* NaN = not given */
  const float* norm_dev; /* device scalar or NULL */
} orlhf_norm;

/* Bytes of workspace the per-token reductions need for an [n_rows, n_cols] problem. */
int64_t orlhf_token_workspace_bytes(int64_t n_rows, int64_t n_cols);

/*
 * Masked aggregation of a per-token fp32 matrix.
 *   TOKEN_MEAN / SEQ_MEAN: aggregate_loss (openrlhf/models/loss.py:11-39) and masked_mean with
 *   dim=None (openrlhf/models/utils.py:166-169); out = 1 float.
 *   ROW_MEAN: masked_mean with dim=-1; out = n_rows floats; `norm` ignored.
 * row_coef (float [n_rows], nullable) receives d(out)/d(x[b,t]) / mask[b,t] for the backward.
 * An all-zero mask gives NaN (0/0) in TOKEN_MEAN/ROW_MEAN exactly as the reference does.
 */
int orlhf_masked_aggregate_fwd(const float* x, const void* mask, int mask_dtype, int64_t n_rows,
                               int64_t n_cols, const int64_t* cu_seqlens, int mode,
                               const orlhf_norm* norm, void* workspace, float* out,
                               float* row_coef, orlhf_stream_t stream);
/*
 * The loss normalisers of one batch (openrlhf/utils/loss_utils.py:33-47,66-74): out2[0] =
 * sum(mask) (batch_num_tokens before its all-reduce), out2[1] = number of rows whose mask sum is
 * > 0 (global_batch_size before its all-reduce). fp64 accumulation, fp32 out.
 */
int orlhf_mask_counts(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                      const int64_t* cu_seqlens, void* workspace, float* out2, orlhf_stream_t stream);

/*
 * row_coef alone, from the mask: the weight of row b's masked token sum in aggregate_loss
 * (openrlhf/models/loss.py:11-39) for TOKEN_MEAN / SEQ_MEAN (/ SEQ_MEAN_TOKEN_SUM), known before
 * any loss value is, which is what lets the fused actor step differentiate in its single pass.
 * Padded layout. workspace: orlhf_token_workspace_bytes(n_rows, n_cols).
 */
int orlhf_mask_row_coef(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols, int mode,
                        const orlhf_norm* norm, void* workspace, float* row_coef, orlhf_stream_t stream);

/* g_x[b,t] = g(b) * row_coef[b] * mask[b,t]; g(b) = g_out[0] (scalar modes) or g_out[b]. */
int orlhf_masked_aggregate_bwd(const float* g_out, const void* mask, int mask_dtype,
                               int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens, int mode,
                               const float* row_coef, float* g_x, orlhf_stream_t stream);

typedef struct orlhf_policy_params {
  float clip_eps_low, clip_eps_high;
  float dual_clip;    /* <= 0: no dual clip */
  int policy_type;    /* orlhf_policy_type */
  int is_correction;  /* orlhf_is_correction (needs rollout_log_probs) */
  float is_low, is_high;
  int token_level;    /* 1: TOKEN_MEAN, 0: SEQ_MEAN (GSPO forces 0, loss.py:143-144) */
  orlhf_norm norm;
} orlhf_policy_params;

/*
 * PolicyLoss.forward (openrlhf/models/loss.py:157-230): PPO / GSPO surrogate with low/high clip,
 * dual clip, TIS / ICEPOP / seq-mask-TIS importance correction and token- or sequence-level
 * aggregation. All per-token inputs fp32 in the row layout above; rollout_log_probs nullable.
 *   out4     float [4]: loss, clip_ratio, ppo_kl, vllm_kl (NaN when no correction is applied)
 *   row_coef float [n_rows]: aggregation weight per row (for the backward)
 *   row_aux  float [n_rows, 2]: {GSPO sequence ratio or seq-mask-TIS 0/1 row flag,
 *            1/max(sum(mask), 1)}; written only in those two modes, always required
 */
int orlhf_policy_loss_fwd(const float* log_probs, const float* old_log_probs,
                          const float* advantages, const void* mask, int mask_dtype,
                          const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                          const int64_t* cu_seqlens, const orlhf_policy_params* params,
                          void* workspace, float* out4, float* row_coef, float* row_aux,
                          orlhf_stream_t stream);
/*
 * The same forward that also writes g_log_probs = d out4[0] / d log_probs (upstream gradient 1) in
 * the same pass: 4 more bytes per token instead of the 21 of orlhf_policy_loss_bwd, bit-identical
 * to what that writes for g_out = 1. Only where a token's weight is known before the pass: PPO,
 * token_level = 1 and a given count in params->norm (what the trainer passes as batch_num_tokens,
 * openrlhf/trainer/ray/ppo_actor.py:306-318); anything else is ORLHF_ERR_INVALID_ARG.
 * No reference counterpart (the reference leaves the backward to autograd).
 */
int orlhf_policy_loss_fwd_grad(const float* log_probs, const float* old_log_probs,
                               const float* advantages, const void* mask, int mask_dtype,
                               const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                               const int64_t* cu_seqlens, const orlhf_policy_params* params,
                               void* workspace, float* out4, float* row_coef, float* row_aux,
                               float* g_log_probs, orlhf_stream_t stream);
/*
 * orlhf_policy_loss_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same
 * results, bit for bit, with the partial sums in a scratch array built into the library
 * (ORLHF_NOALLOC_SCRATCH_BYTES per GPU, held from the first call on that GPU until the process
 * ends) instead of a caller's workspace. It calls no hipMalloc / hipFree and no allocating
 * routine. No counterpart in the reference. Problems whose orlhf_token_workspace_bytes(n_rows,
 * n_cols) exceeds the scratch return ORLHF_ERR_UNSUPPORTED. All calls on one GPU share that GPU's
 * scratch: calls that overlap on one GPU (different streams or host threads) race; serialise them.
 * `stream` has to belong to the current device (ORLHF_ERR_INVALID_ARG otherwise: the scratch is
 * the current device's). The first call on a device looks the scratch up (hipGetSymbolAddress) and
 * has to come outside stream capture; every later call on that device may be captured.
 */
#define ORLHF_NOALLOC_SCRATCH_BYTES (8 << 20)
int orlhf_policy_loss_fwd_noalloc(const float* log_probs, const float* old_log_probs,
                                  const float* advantages, const void* mask, int mask_dtype,
                                  const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                                  const int64_t* cu_seqlens, const orlhf_policy_params* params,
                                  float* out4, float* row_coef, float* row_aux,
                                  orlhf_stream_t stream);
/* grad wrt log_probs only (everything else is detached in the callers). g_out: device scalar.
 * workspace (orlhf_token_workspace_bytes) is used by GSPO only and may be NULL otherwise. */
int orlhf_policy_loss_bwd(const float* g_out, const float* log_probs, const float* old_log_probs,
                          const float* advantages, const void* mask, int mask_dtype,
                          const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                          const int64_t* cu_seqlens, const orlhf_policy_params* params,
                          const float* row_coef, const float* row_aux, void* workspace,
                          float* g_log_probs, orlhf_stream_t stream);

/*
 * ValueLoss.forward (openrlhf/models/loss.py:244-269): 0.5 * aggregate(max((vc-R)^2, (v-R)^2)),
 * vc = old + clamp(v - old, -eps, eps); has_clip == 0 gives 0.5 * aggregate((v-R)^2).
 *   out2 float [2]: loss, masked mean of the values (the "values" status of
 *   openrlhf/trainer/ray/ppo_critic.py:174, from the same pass)
 */
int orlhf_value_loss_fwd(const float* values, const float* old_values, const float* returns,
                         const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                         const int64_t* cu_seqlens, int has_clip, float clip_eps, int token_level,
                         const orlhf_norm* norm, void* workspace, float* out2, float* row_coef,
                         orlhf_stream_t stream);
/* Forward plus g_values = d out2[0] / d values in one pass; token mean over a given count only
 * (see orlhf_policy_loss_fwd_grad). No reference counterpart. */
int orlhf_value_loss_fwd_grad(const float* values, const float* old_values, const float* returns,
                              const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                              const int64_t* cu_seqlens, int has_clip, float clip_eps,
                              const orlhf_norm* norm, void* workspace, float* out2, float* row_coef,
                              float* g_values, orlhf_stream_t stream);
int orlhf_value_loss_bwd(const float* g_out, const float* values, const float* old_values,
                         const float* returns, const void* mask, int mask_dtype, int64_t n_rows,
                         int64_t n_cols, const int64_t* cu_seqlens, int has_clip, float clip_eps,
                         const float* row_coef, float* g_values, orlhf_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Advantage kernels (forward only; the reference runs them under torch.no_grad())
 * ---------------------------------------------------------------------------------------- */

/*
 * compute_reward (openrlhf/models/utils.py:98-126): reward[b,t] = -max(kl_coef,0)*kl[b,t]
 * + clamp(r[b]) at the row's last position whose (int64)mask is maximal (= last 1; last column
 * for an all-zero row). eos_index (int64 [n_rows], nullable) receives that column.
 */
int orlhf_compute_reward(const float* r, float kl_coef, const float* kl, const void* mask,
                         int mask_dtype, int64_t n_rows, int64_t n_cols,
                         const int64_t* cu_seqlens, int has_clip, float clip_low, float clip_high,
                         float* reward, int64_t* eos_index, orlhf_stream_t stream);

/*
 * get_advantages_and_returns (openrlhf/trainer/ppo_utils/experience_maker.py:332-377):
 * v = m*values, r = m*rewards, delta_t = r_t + gamma*v_{t+1} - v_t, A_t = delta_t +
 * gamma*lambd*A_{t+1}, returns = A + v; every column takes part and nothing is re-masked.
 * Parallel reverse scan per row, fp64 carries.
 * row_order (int64 [n_rows], nullable; also in the two scans below): a permutation of the rows;
 * workgroup slot s walks row row_order[s]. Results do not depend on it; a caller that knows the
 * row lengths of a ragged packed batch passes the rows longest first, so that no long row's
 * sequential walk is left running alone at the end of the launch. The kernels trust it to be a
 * permutation: an entry outside [0, n_rows) is skipped, a row named twice is computed twice (to the
 * same values), and a row that no entry names keeps whatever its outputs held. A caller that
 * cannot vouch for it (the library's own Python wrappers build it with a sort of the lengths)
 * passes NULL.
 */
int orlhf_gae_scan(const float* values, const float* rewards, const void* mask, int mask_dtype,
                   int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                   const int64_t* row_order, float gamma, float lambd, float* advantages,
                   float* returns, orlhf_stream_t stream);

/* get_cumulative_returns (experience_maker.py:379-411): G_t = m_t*r_t + gamma*G_{t+1}. */
int orlhf_discounted_returns(const float* rewards, const void* mask, int mask_dtype,
                             int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                             const int64_t* row_order, float gamma, float* returns,
                             orlhf_stream_t stream);

/*
 * The per-experience body of compute_advantages_and_returns (experience_maker.py:276-312) in one
 * pass: compute_reward (openrlhf/models/utils.py:98-126) followed by get_advantages_and_returns
 * (values and advantages given) or get_cumulative_returns (both NULL), without the per-token
 * reward ever being stored. Per row: the last maximal mask position is found, then the reverse
 * scan makes each token reward -max(kl_coef, 0)*kl[t] (+ the clipped r[b] at that position) as
 * it loads kl. reward_sum[b] (nullable) = the row's token rewards summed over every column,
 * which is the reference's info["return"] (experience_maker.py:311). Results equal
 * orlhf_compute_reward followed by orlhf_gae_scan / orlhf_discounted_returns bit for bit.
 */
int orlhf_reward_scan(const float* r, float kl_coef, const float* kl, const float* values,
                      const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                      const int64_t* cu_seqlens, const int64_t* row_order, int has_clip,
                      float clip_low, float clip_high, float gamma, float lambd, float* advantages,
                      float* returns, float* reward_sum, orlhf_stream_t stream);

/*
 * Group baseline / normalisation of scalar rewards (experience_maker.py:246-272).
 * rewards / out / group_std are in experience order; indices[i] (int64, nullable = identity) is
 * the prompt-order slot of sample i, so group g holds slots g*n .. g*n+n-1. group_std
 * (nullable) receives the unbiased std of each sample's group (NaN for n == 1, as torch.std).
 */
int orlhf_group_normalize(const float* rewards, const int64_t* indices, int64_t n_prompts,
                          int64_t n_samples, int estimator, float* out, float* group_std,
                          void* workspace /* n_prompts*n_samples floats */, orlhf_stream_t stream);

/*
 * Global masked whitening (experience_maker.py:314-328) over a flat array of n elements:
 * mean = sum(x*m)/sum(m); var = sum((x-mean)^2*m)/sum(m); rstd = rsqrt(max(var,1e-8)) or 1 when
 * std_norm == 0; out = (x - mean)*rstd at EVERY position, masked or not. out may alias x.
 * stats (float [2], nullable) receives mean and rstd. workspace: orlhf_whiten_workspace_bytes(n).
 */
int64_t orlhf_whiten_workspace_bytes(int64_t n);
int orlhf_masked_whiten(const float* x, const void* mask, int mask_dtype, int64_t n, int std_norm,
                        void* workspace, float* out, float* stats, orlhf_stream_t stream);

/*
 * The same whitening over a list of blocks (one per experience, as the reference holds them in
 * experience_maker.py:314-328) without gathering them into one array first: xs / masks / outs
 * are HOST arrays of n_blocks device pointers, ns the element counts; all masks share
 * mask_dtype. Statistics are taken over all blocks together. outs[i] may alias xs[i].
 * workspace: orlhf_whiten_multi_workspace_bytes(ns, n_blocks).
 */
int64_t orlhf_whiten_multi_workspace_bytes(const int64_t* ns, int n_blocks);
int orlhf_masked_whiten_multi(const float* const* xs, const void* const* masks, int mask_dtype,
                              const int64_t* ns, int n_blocks, int std_norm, void* workspace,
                              float* const* outs, float* stats, orlhf_stream_t stream);

/*
 * The KL block of experience making (openrlhf/trainer/ppo_utils/experience_maker.py:202-216) in
 * one pass: kl = compute_approx_kl(log_probs, log_probs_base, estimator) (float, nullable),
 * kl_mean[b] = masked_mean(kl, mask, dim=-1), diff_mean[b] = masked_mean(log_probs -
 * log_probs_base, mask, dim=-1) (float [n_rows], each nullable; an empty row gives NaN as the
 * reference's 0/0). enabled == 0 is the branch without a reference model: kl and both
 * differences are zeros and the log-prob pointers are not read. Inputs of `dtype`, fp32 maths.
 */
int orlhf_kl_rows(const void* log_probs, const void* log_probs_base, int dtype, const void* mask,
                  int mask_dtype, int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                  int estimator, int enabled, float* kl, float* kl_mean, float* diff_mean,
                  orlhf_stream_t stream);

/*
 * masked_normalize (openrlhf/models/utils.py:172-179) over each row: mean = sum(x*m)/max(sum(m),1),
 * c = (x - mean)*m, var = sum(c^2)/max(sum(m),1), out = c * rsqrt(max(var, eps)). out may alias x.
 */
int orlhf_masked_normalize_rows(const float* x, const void* mask, int mask_dtype, int64_t n_rows,
                                int64_t n_cols, const int64_t* cu_seqlens, float eps, float* out,
                                orlhf_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Sequence-level pieces of the preference trainers (the callers next to the hot path).
 * ------------------------------------------------------------------------------------------ */

/*
 * DPOTrainer._get_batch_logps (openrlhf/trainer/dpo_trainer.py:362-382): per-sequence sum and
 * mean of per-token log-probs [n_rows, n_cols] (n_cols = T-1) under the loss mask
 *   m[b,t] = attention_mask[b,t+1] != 0  and  t+1 >= prompt_id_lens[b]
 * built on the fly from attention_mask [n_rows, n_cols+1] (mask dtype as elsewhere; NONE = all
 * ones) and prompt_id_lens (int64 [n_rows], nullable = no prompt masking); the reference clones
 * the mask, clears it row by row from Python and shifts it. sums / means / counts (float
 * [n_rows], each nullable): sum(lp*m), that sum / sum(m) (NaN when no loss token, as torch) and
 * sum(m) (keep it for the backward).
 */
int orlhf_sequence_logps_fwd(const float* per_token_logps, const void* attention_mask, int mask_dtype,
                             const int64_t* prompt_id_lens, int64_t n_rows, int64_t n_cols,
                             float* sums, float* means, float* counts, orlhf_stream_t stream);
/* g_per_token[b,t] = m[b,t] * (g_sums[b] + g_means[b] / counts[b]); g_sums / g_means nullable. */
int orlhf_sequence_logps_bwd(const float* g_sums, const float* g_means, const void* attention_mask,
                             int mask_dtype, const int64_t* prompt_id_lens, const float* counts,
                             int64_t n_rows, int64_t n_cols, float* g_per_token,
                             orlhf_stream_t stream);

/*
 * Pairwise losses over n (chosen, rejected) scalars, mean over pairs (NaN for n == 0):
 * DPOLoss (openrlhf/models/loss.py:300-335), PairWiseLoss (:272-284), LogExpLoss (:287-297).
 * logit z = (chosen - rejected) - (ref_chosen - ref_rejected); ref_chosen / ref_rejected are
 * nullable (0): for PairWiseLoss pass the margin as ref_chosen. kind: enum orlhf_pair_loss.
 *   DPO_SIGMOID: -logsigmoid(beta z)(1 - label_smoothing) - logsigmoid(-beta z) label_smoothing
 *   DPO_IPO: (z - 1/(2 beta))^2      LOGSIGMOID: -logsigmoid(z)      LOGEXP: log(1 + exp(-z))
 * chosen_rewards / rejected_rewards (float [n], nullable): beta*(chosen - ref_chosen) and
 * beta*(rejected - ref_rejected), the detached reward estimates DPOLoss returns.
 */
int orlhf_pair_loss_fwd(const float* chosen, const float* rejected, const float* ref_chosen,
                        const float* ref_rejected, int64_t n, int kind, double beta,
                        double label_smoothing, float* loss, float* chosen_rewards,
                        float* rejected_rewards, orlhf_stream_t stream);
/* g_chosen = g_out[0]/n * dloss/dz, g_rejected = -g_chosen (each nullable). */
int orlhf_pair_loss_bwd(const float* g_out, const float* chosen, const float* rejected,
                        const float* ref_chosen, const float* ref_rejected, int64_t n, int kind,
                        double beta, double label_smoothing, float* g_chosen, float* g_rejected,
                        orlhf_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Row layouts: padded [n_rows, n_cols] + mask  <->  packed flat tokens + cu_seqlens. Index work
 * and copies, bit-exact. The per-token entry points above take either layout.
 * ------------------------------------------------------------------------------------------ */

/*
 * Per mask row: first = first non-zero column (n_cols if none), end = one past the last non-zero
 * column (0 if none), length = end - first (0 if none); each output int64 [n_rows], nullable.
 * Right-padded rows: length is what remove_padding_in_sequences keeps
 * (openrlhf/trainer/ppo_utils/experience.py:236-247, attention_mask.flip(0).argmax()); interior
 * zeros stay inside the extent.
 */
int orlhf_row_extents(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                      int64_t* first, int64_t* end, int64_t* length, orlhf_stream_t stream);

/* cu_seqlens[0] = 0, cu_seqlens[i+1] = cu_seqlens[i] + lengths[i] (int64 [n_rows+1]): the
 * boundaries flash-attn's unpad_input returns (openrlhf/models/ring_attn_utils.py:129-140). */
int orlhf_cu_seqlens(const int64_t* lengths, int64_t n_rows, int64_t* cu_seqlens,
                     orlhf_stream_t stream);

/* dst[cu[b] + j] = src[b, first[b] + j] for j < cu[b+1] - cu[b]; first nullable (0). Elements
 * are elem_bytes (1, 2, 4, 8) wide and copied as bits. */
int orlhf_pack_rows(const void* src, int elem_bytes, int64_t n_rows, int64_t n_cols,
                    const int64_t* first, const int64_t* cu_seqlens, void* dst,
                    orlhf_stream_t stream);

/* orlhf_pack_rows for several fields that share n_rows, n_cols, first and cu_seqlens, in one launch
 * per eight fields (a rollout batch packs four to ten per-token tensors over the same mask:
 * openrlhf/trainer/ppo_utils/experience.py:199-247 slices every field of every sample). `fields` is a
 * HOST array of n_fields entries; the pointers inside are device pointers. */
typedef struct orlhf_pack_field {
  const void* src; /* [n_rows, n_cols] elements of elem_bytes */
  void* dst;       /* cu_seqlens[n_rows] elements */
  int elem_bytes;  /* 1, 2, 4 or 8 */
} orlhf_pack_field;
int orlhf_pack_rows_multi(const orlhf_pack_field* fields, int n_fields, int64_t n_rows, int64_t n_cols,
                          const int64_t* first, const int64_t* cu_seqlens, orlhf_stream_t stream);

/* dst[cu[b] + j] = src[src_start[b] + j] for j < cu[b+1] - cu[b]: rows picked out of a packed
 * array into a new packed array, in any order and with repeats (a replay buffer handing out a
 * micro-batch without going through the padded form of
 * openrlhf/trainer/ppo_utils/experience.py:199-247). max_len bounds the row lengths (it sizes the
 * launch; rows longer than it are cut). Elements are elem_bytes (1, 2, 4, 8) wide. */
int orlhf_gather_rows(const void* src, int elem_bytes, int64_t n_rows, int64_t max_len,
                      const int64_t* src_start, const int64_t* cu_seqlens, void* dst,
                      orlhf_stream_t stream);

/*
 * zero_pad_sequences(..., side, value, stack=True) (openrlhf/utils/utils.py:93-106) from the
 * packed layout: dst [n_rows, n_cols] is filled with fill_bits (low elem_bytes bytes) and row b
 * receives src[cu[b] .. cu[b+1]) at its right end (left_side = 1: padding on the left) or at
 * its left end (left_side = 0). Rows longer than n_cols are cut.
 */
int orlhf_pad_rows(const void* src, int elem_bytes, const int64_t* cu_seqlens, int64_t n_rows,
                   int64_t n_cols, int left_side, uint64_t fill_bits, void* dst,
                   orlhf_stream_t stream);

/*
 * The unpadding in front of the packed model forward, unpad_and_slice_tensor on one GPU
 * (openrlhf/models/ring_attn_utils.py:129-140), which calls unpad_input / index_first_axis of
 * flash-attn 2.8.3 (flash_attn/bert_padding.py, not in the reference tree; its published
 * algorithm: indices = nonzero(mask.flatten()), seqlens = mask.sum(-1), cu_seqlens =
 * pad(cumsum(seqlens), (1, 0)), gathers by indices), for masks of zeros and ones with the ones
 * anywhere in a row (left padding, right padding, holes).
 *
 * orlhf_mask_row_counts: counts[b] = number of non-zero columns of mask row b (seqlens_in_batch;
 *   orlhf_cu_seqlens turns them into cu_seqlens). tile_counts (int32 [n_rows, ceil(n_cols /
 *   ORLHF_UNPAD_TILE)], nullable): the same per tile of ORLHF_UNPAD_TILE columns, from the same pass.
 * orlhf_unpad_sequences: for the r-th non-zero column t of row b, at slot cu_seqlens[b] + r of each
 *   output that is not NULL:
 *     indices          b * n_cols + t                      (unpad_input's indices)
 *     packed_sequences sequences[b, t]                     (:130-131)
 *     rolled_sequences sequences[b, (t + 1) mod n_cols]    (torch.roll(sequences, -1, 1), :129,132-136)
 *     position_ids     r                                   (clip(cumsum(mask, -1) - 1, min=0), :137-140)
 *   sequences may be NULL when neither sequence output is asked for. capacity is the number of
 *   slots each output holds (cu_seqlens[n_rows] when they are sized exactly); slots past it are
 *   not written. tile_counts: what orlhf_mask_row_counts wrote for the same mask, or NULL. With it
 *   every (row, tile) is a work item of its own that knows its first slot (tiles without attended
 *   columns cost nothing and fully attended ones do not read the mask); without it a workgroup
 *   walks a whole row, tile after tile. Same outputs either way.
 */
#define ORLHF_UNPAD_TILE 2048
int orlhf_mask_row_counts(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                          int64_t* counts, int32_t* tile_counts, orlhf_stream_t stream);
int orlhf_unpad_sequences(const int64_t* sequences, const void* mask, int mask_dtype,
                          int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                          const int32_t* tile_counts, int64_t capacity, int64_t* indices,
                          int64_t* packed_sequences, int64_t* rolled_sequences, int64_t* position_ids,
                          orlhf_stream_t stream);

/*
 * The way back, gather_and_pad_tensor on one GPU (openrlhf/models/ring_attn_utils.py:181, which is
 * flash-attn's pad_input: zeros, then output[indices] = input): dst holds n_dst rows of `inner`
 * elements of elem_bytes (1, 2, 4, 8) bytes, all set to zero, then row indices[i] receives row i
 * of src (n rows). dst must be 16-byte aligned; an index outside [0, n_dst) is skipped.
 */
int orlhf_pad_by_indices(const void* src, int elem_bytes, int64_t n, int64_t inner,
                         const int64_t* indices, int64_t n_dst, void* dst, orlhf_stream_t stream);

/*
 * The inverse, flash-attn's index_first_axis (what unpad_input applies to every per-token tensor,
 * openrlhf/models/ring_attn_utils.py:130-140, and the gradient of pad_input): row i of dst (n rows
 * of `inner` elements) = row indices[i] of src (n_src rows); an index outside [0, n_src) gives a
 * row of zeros.
 */
int orlhf_gather_by_indices(const void* src, int elem_bytes, int64_t n_src, int64_t inner,
                            const int64_t* indices, int64_t n, void* dst, orlhf_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Diagnostics. Not part of the reference-citing interface above: nothing of the reference maps to
 * these two; they exist so that the matrix-core tile the lm-head entry points are built on can be
 * tested and timed on its own (bench.py --workload matrix_tile, tests/test_gpu_matrix_tile.py).
 * ------------------------------------------------------------------------------------------ */

/*
 * c [m, n] (fp32, row stride ldc) = or += a * b^T through that tile, one 256 x 256 tile per
 * workgroup: a is [m, k] with row stride lda (a_mn_major = 0) or stored as [k, m] with row stride
 * lda (a_mn_major = 1); b likewise with n. accumulate != 0 continues the sums found in c inside the
 * accumulators (the same bits as one product over the concatenated depth). bf16 or fp16 operands,
 * 4-byte aligned bases, even row strides below 2^23.
 */
int orlhf_matrix_tile_product(const void* a, const void* b, int dtype, int64_t m, int64_t n, int64_t k,
                              int64_t lda, int64_t ldb, int a_mn_major, int b_mn_major, int accumulate,
                              float* c, int64_t ldc, orlhf_stream_t stream);

/*
 * The plain product of two K-major operands,
 * a [m, k] (row stride lda) and b [n, k] (row stride ldb), bf16 or fp16, through the matrix-core
 * tile the lm-head entry points above are built on, one 256 x 256 tile per workgroup. Nothing but
 * the product is done: thread t of tile (i, j) leaves the sum of its 256 accumulators in
 * tile_sums[(i * ceil(n / 256) + j) * 256 + t] (float, ceil(m / 256) * ceil(n / 256) * 256
 * entries), so the 256 sums of a tile add up to the sum of that block of a * b^T. With
 * resident_operands != 0 the steady loop loads nothing (every slab is multiplied out of what the
 * LDS buffers hold after the first two slabs; the sums are meaningless): the time of that run is
 * what the same LDS reads, MFMAs and barriers take on their own, the ceiling the tile can be read
 * against on a given GPU and clock. A row stride of 0 makes every row of that operand its first
 * row (all loads of the steady loop then hit the L1: the cost of issuing them and writing LDS,
 * without the cost of fetching). Operands need 4-byte aligned bases and even row strides.
 */
int orlhf_matrix_tile_probe(const void* a, const void* b, int dtype, int64_t m, int64_t n, int64_t k,
                            int64_t lda, int64_t ldb, int resident_operands, float* tile_sums,
                            orlhf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* OPENRLHF_AMD_H */
