// Index work around the one-pass PPO actor step: the per-token terms live in [B, A] tensors
// (action columns of a padded batch), the vocabulary-row kernel wants one value per logits row
// ([B*T] rows, or the packed rows of the attended tokens). One gather kernel builds every per-row
// array the step needs (labels, row mask, old / advantage / rollout / base log-probs, aggregation
// weights), and one reduction produces every loss value of the step from the per-row results and
// scatters the action log-probs / entropy back to [B, A].
#include "token_terms.h"

namespace orlhf {

struct ActorRowsIn {
  const int64_t* sequences;       // [B, T]
  const void* mask;               // [B, A]
  const int64_t* packed_indices;  // [n_rows] flat positions in the [B, T] grid, or NULL: row r is position r
  const float *old_lp, *adv, *rollout, *base;  // [B, A]; rollout / base nullable
  const float *row_coef_policy, *row_coef_token;  // [B]
  int64_t batch, seqlen, width, n_rows;
  float loss_scale;
};

struct ActorRowsOut {
  int64_t* labels;
  uint8_t* need;
  float *weight, *old_lp, *adv, *rollout, *base, *policy_coef, *token_coef;  // [n_rows]; rollout / base nullable
};

// Row r of the logits is position (b, t) of the padded batch; its action column is t - (T - 1 - A).
__device__ __forceinline__ bool row_position(const int64_t* packed_indices, int64_t r, int64_t seqlen, int64_t width,
                                             int64_t& b, int64_t& t, int64_t& col) {
  const int64_t flat = packed_indices != nullptr ? packed_indices[r] : r;
  b = flat / seqlen;
  t = flat - b * seqlen;
  col = t - (seqlen - 1 - width);
  return col >= 0 && col < width;
}

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void actor_rows_gather_kernel(ActorRowsIn in, ActorRowsOut out) {
  for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < in.n_rows; r += (int64_t)gridDim.x * kBlock) {
    int64_t b, t, col;
    const bool inside = row_position(in.packed_indices, r, in.seqlen, in.width, b, t, col);
    // the label of position t is the next token of the same padded row (the row rolled left by one)
    out.labels[r] = in.sequences[b * in.seqlen + (t + 1 == in.seqlen ? 0 : t + 1)];
    const int64_t i = b * in.width + col;
    const float m = inside ? load_mask<MASK_DT>(in.mask, i) : 0.0f;
    out.need[r] = m != 0.0f ? 1 : 0;
    out.weight[r] = m;
    out.old_lp[r] = inside ? in.old_lp[i] : 0.0f;
    out.adv[r] = inside ? in.adv[i] : 0.0f;
    if (out.rollout != nullptr) out.rollout[r] = inside ? in.rollout[i] : 0.0f;
    if (out.base != nullptr) out.base[r] = inside ? in.base[i] : 0.0f;
    out.policy_coef[r] = inside ? in.row_coef_policy[b] * m * in.loss_scale : 0.0f;
    out.token_coef[r] = inside ? in.row_coef_token[b] * m * in.loss_scale : 0.0f;
  }
}

// ---------------------------------------------------------------- loss values from the per-row results
struct ActorValuesIn {
  const float *logprob, *entropy;  // [n_rows] from the one-pass kernel; entropy nullable
  const float *weight, *old_lp, *adv, *rollout, *base, *policy_coef, *token_coef;  // [n_rows]
  const int64_t* packed_indices;
  int64_t seqlen, width, n_rows;
  PolicyTok pol;
  int kl_estimator;
  float kl_coef, entropy_coef, loss_scale;
  int entropy_in_loss;
};

constexpr int kValQ = 8;  // policy, kl, entropy (coefficient-weighted), sum w, w*clipped, w*(old-lp), w*(rollout-old), w*(lp-base)
constexpr int kValBlock = 1024;

__global__ __launch_bounds__(kValBlock) void actor_values_partial_kernel(ActorValuesIn in, double* __restrict__ partial,
                                                                         float* __restrict__ action_log_probs,
                                                                         float* __restrict__ action_entropy) {
  __shared__ double lds[kValQ][kValBlock / kWave];
  double acc[kValQ];
#pragma unroll
  for (int q = 0; q < kValQ; ++q) acc[q] = 0.0;
  const int64_t r = (int64_t)blockIdx.x * kValBlock + threadIdx.x;
  if (r < in.n_rows) {
    const float w = in.weight[r];
    int64_t b, t, col;
    const bool inside = row_position(in.packed_indices, r, in.seqlen, in.width, b, t, col);
    const float lp = in.logprob[r] * w;  // action_log_probs = log_probs * action_mask
    if (inside) {
      action_log_probs[b * in.width + col] = lp;
      if (action_entropy != nullptr) action_entropy[b * in.width + col] = in.entropy[r];
    }
    if (w != 0.0f) {
      const float old_v = in.old_lp[r], roll_v = in.rollout != nullptr ? in.rollout[r] : 0.0f;
      const float v[4] = {lp, old_v, in.adv[r], roll_v};
      float q[PolicyTok::kQ];
      in.pol.eval(0, v, w, q);  // {loss*w, w, clipped*w, (old-lp)*w, (rollout-old)*w}
      acc[0] = (double)in.policy_coef[r] * (double)(q[0] / w);
      if (in.base != nullptr) {
        const float d = lp - in.base[r];
        float kv, kd;
        kl_value(in.kl_estimator, d, kv, kd);
        acc[1] = (double)in.token_coef[r] * (double)kv;
        acc[7] = (double)(d * w);
      }
      if (in.entropy != nullptr) acc[2] = (double)in.token_coef[r] * (double)in.entropy[r];
      acc[3] = (double)q[1];
      acc[4] = (double)q[2];
      acc[5] = (double)q[3];
      acc[6] = (double)q[4];
    }
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
#pragma unroll
    for (int q = 0; q < kValQ; ++q) acc[q] += __shfl_xor(acc[q], o, kWave);
  }
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
    for (int q = 0; q < kValQ; ++q) lds[q][wave] = acc[q];
  }
  __syncthreads();
  if (threadIdx.x < kValQ) {
    double s = 0.0;
    for (int w = 0; w < kValBlock / kWave; ++w) s += lds[threadIdx.x][w];
    partial[(int64_t)blockIdx.x * kValQ + threadIdx.x] = s;
  }
}

// out[0..7] = loss, actor_loss, clip_ratio, ppo_kl, vllm_kl, kl_loss, entropy_loss, logprobs_diff
__global__ __launch_bounds__(kBlock) void actor_values_final_kernel(const double* __restrict__ partial, int64_t n_blocks,
                                                                    double loss_scale, float kl_coef, float entropy_coef,
                                                                    int has_base, int has_entropy, int entropy_in_loss,
                                                                    int has_rollout, float* __restrict__ out) {
  __shared__ double lds[kValQ][kWavesPerBlock];
  double acc[kValQ];
#pragma unroll
  for (int q = 0; q < kValQ; ++q) acc[q] = 0.0;
  for (int64_t i = threadIdx.x; i < n_blocks; i += kBlock) {
#pragma unroll
    for (int q = 0; q < kValQ; ++q) acc[q] += partial[i * kValQ + q];
  }
#pragma unroll
  for (int q = 0; q < kValQ; ++q) acc[q] = block_sum(acc[q], lds[q]);
  if (threadIdx.x == 0) {
    const double actor = acc[0] / loss_scale, kl = acc[1] / loss_scale, ent = acc[2] / loss_scale, n = acc[3];
    double loss = actor;
    if (has_base) loss += kl * (double)kl_coef;
    if (has_entropy && entropy_in_loss) loss -= ent * (double)entropy_coef;
    out[0] = (float)loss;
    out[1] = (float)actor;
    out[2] = (float)(acc[4] / n);
    out[3] = (float)(acc[5] / n);
    out[4] = has_rollout ? (float)(acc[6] / n) : NAN;
    out[5] = has_base ? (float)kl : NAN;
    out[6] = has_entropy ? (float)ent : NAN;
    out[7] = has_base ? (float)(acc[7] / n) : NAN;
  }
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_actor_step_gather(const int64_t* sequences, const void* action_mask, int mask_dtype,
                                       const int64_t* packed_indices, int64_t batch, int64_t seqlen, int64_t width,
                                       int64_t n_rows, const float* old_log_probs, const float* advantages,
                                       const float* rollout_log_probs, const float* base_log_probs,
                                       const float* row_coef_policy, const float* row_coef_token, float loss_scale,
                                       int64_t* labels_rows, uint8_t* need_rows, float* weight_rows, float* old_rows,
                                       float* adv_rows, float* rollout_rows, float* base_rows, float* policy_coef_rows,
                                       float* token_coef_rows, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(batch >= 0 && seqlen >= 1 && width >= 0 && width <= seqlen - 1 && n_rows >= 0,
                  "actor_step_gather: batch=%lld seqlen=%lld width=%lld n_rows=%lld", (long long)batch, (long long)seqlen,
                  (long long)width, (long long)n_rows);
  ORLHF_CHECK_ARG(packed_indices != nullptr || n_rows == batch * seqlen,
                  "actor_step_gather: %lld rows for a %lld x %lld batch without packed_indices", (long long)n_rows,
                  (long long)batch, (long long)seqlen);
  ORLHF_CHECK_ARG(mask_dtype >= ORLHF_MASK_U8 && mask_dtype <= ORLHF_MASK_I64, "actor_step_gather: unknown mask dtype %d", mask_dtype);
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(sequences && action_mask && old_log_probs && advantages && row_coef_policy && row_coef_token,
                  "actor_step_gather: NULL input");
  ORLHF_CHECK_ARG(labels_rows && need_rows && weight_rows && old_rows && adv_rows && policy_coef_rows && token_coef_rows,
                  "actor_step_gather: NULL output");
  ORLHF_CHECK_ARG((rollout_rows == nullptr) == (rollout_log_probs == nullptr) && (base_rows == nullptr) == (base_log_probs == nullptr),
                  "actor_step_gather: rollout / base inputs and outputs must be given together");
  const ActorRowsIn in{sequences, action_mask, packed_indices, old_log_probs, advantages, rollout_log_probs, base_log_probs,
                       row_coef_policy, row_coef_token, batch, seqlen, width, n_rows, loss_scale};
  const ActorRowsOut out{labels_rows, need_rows, weight_rows, old_rows, adv_rows, rollout_rows, base_rows, policy_coef_rows,
                         token_coef_rows};
  const dim3 grid(flat_grid(n_rows, 4096)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_GATHER(M) hipLaunchKernelGGL(actor_rows_gather_kernel<M>, grid, block, 0, s, in, out)
  switch (mask_dtype) {
    case ORLHF_MASK_U8: ORLHF_GATHER(ORLHF_MASK_U8); break;
    case ORLHF_MASK_F32: ORLHF_GATHER(ORLHF_MASK_F32); break;
    default: ORLHF_GATHER(ORLHF_MASK_I64); break;
  }
#undef ORLHF_GATHER
  ORLHF_CHECK_LAUNCH("orlhf_actor_step_gather");
  return ORLHF_OK;
}

extern "C" int64_t orlhf_actor_step_values_workspace_bytes(int64_t n_rows) {
  const int64_t blocks = n_rows > 0 ? (n_rows + kValBlock - 1) / kValBlock : 1;
  return blocks * kValQ * (int64_t)sizeof(double);
}

extern "C" int orlhf_actor_step_values(const float* logprob_rows, const float* entropy_rows, const float* weight_rows,
                                       const float* old_rows, const float* adv_rows, const float* rollout_rows,
                                       const float* base_rows, const float* policy_coef_rows,
                                       const float* token_coef_rows, const int64_t* packed_indices, int64_t seqlen,
                                       int64_t width, int64_t n_rows, const orlhf_step_terms* t, float loss_scale,
                                       int entropy_in_loss, void* workspace, float* action_log_probs,
                                       float* action_entropy, float* out8, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(t != nullptr && out8 != nullptr && workspace != nullptr, "actor_step_values: NULL terms / out / workspace");
  ORLHF_CHECK_ARG(n_rows >= 0 && seqlen >= 1 && width >= 0 && width <= seqlen - 1, "actor_step_values: seqlen=%lld width=%lld n_rows=%lld",
                  (long long)seqlen, (long long)width, (long long)n_rows);
  ORLHF_CHECK_ARG(loss_scale != 0.0f && loss_scale == loss_scale, "actor_step_values: loss_scale must be a non-zero number");
  ORLHF_CHECK_ARG(n_rows == 0 || (logprob_rows && weight_rows && old_rows && adv_rows && policy_coef_rows && token_coef_rows && action_log_probs),
                  "actor_step_values: NULL input");
  ORLHF_CHECK_ARG((entropy_rows == nullptr) == (action_entropy == nullptr), "actor_step_values: entropy rows and output must be given together");
  ORLHF_CHECK_ARG(t->is_correction == ORLHF_IS_NONE || t->is_correction == ORLHF_IS_TIS || t->is_correction == ORLHF_IS_ICEPOP,
                  "actor_step_values: only token-level importance corrections (none, tis, icepop), got %d", t->is_correction);
  ORLHF_CHECK_ARG(t->is_correction == ORLHF_IS_NONE || rollout_rows != nullptr, "actor_step_values: importance correction needs rollout rows");
  ORLHF_CHECK_ARG(base_rows == nullptr || (t->kl_estimator >= ORLHF_KL_K1 && t->kl_estimator <= ORLHF_KL_K3),
                  "actor_step_values: unknown kl_estimator %d", t->kl_estimator);
  ActorValuesIn in{};
  in.logprob = logprob_rows, in.entropy = entropy_rows, in.weight = weight_rows, in.old_lp = old_rows, in.adv = adv_rows;
  in.rollout = rollout_rows, in.base = base_rows, in.policy_coef = policy_coef_rows, in.token_coef = token_coef_rows;
  in.packed_indices = packed_indices, in.seqlen = seqlen, in.width = width, in.n_rows = n_rows;
  in.pol.lp = in.pol.old = in.pol.adv = in.pol.rollout = in.pol.row_aux = nullptr;
  in.pol.lo = 1.0f - t->clip_eps_low;
  in.pol.hi = 1.0f + t->clip_eps_high;
  in.pol.dual = t->dual_clip;
  in.pol.gspo = 0;
  in.pol.is_mode = rollout_rows != nullptr ? t->is_correction : ORLHF_IS_NONE;
  in.pol.is_lo = t->is_low;
  in.pol.is_hi = t->is_high;
  in.kl_estimator = t->kl_estimator;
  in.kl_coef = t->kl_coef, in.entropy_coef = t->entropy_coef, in.loss_scale = loss_scale;
  in.entropy_in_loss = entropy_in_loss;
  const int64_t blocks = n_rows > 0 ? (n_rows + kValBlock - 1) / kValBlock : 0;
  hipStream_t s = (hipStream_t)stream;
  if (blocks > 0) {
    hipLaunchKernelGGL(actor_values_partial_kernel, dim3((unsigned)blocks), dim3(kValBlock), 0, s, in, (double*)workspace,
                       action_log_probs, action_entropy);
    ORLHF_CHECK_LAUNCH("orlhf_actor_step_values(partial)");
  }
  hipLaunchKernelGGL(actor_values_final_kernel, dim3(1), dim3(kBlock), 0, s, (const double*)workspace, blocks,
                     (double)loss_scale, t->kl_coef, t->entropy_coef, base_rows != nullptr ? 1 : 0,
                     entropy_rows != nullptr ? 1 : 0, entropy_in_loss, rollout_rows != nullptr ? 1 : 0, out8);
  ORLHF_CHECK_LAUNCH("orlhf_actor_step_values(final)");
  return ORLHF_OK;
}
