// Per-token loss terms shared by the per-token kernels and by the fused vocabulary-row step:
// the PPO / GSPO surrogate with its derivative and the k1 / k2 / k3 KL estimators.
#pragma once
#include "common.h"

namespace orlhf {

struct PolicyTok {
  static constexpr int kQ = 5;
  const float *lp, *old, *adv, *rollout;
  const float* row_aux;  // [n_rows, 2]
  float lo, hi;          // 1 - eps_low, 1 + eps_high
  float dual;            // <= 0: off
  int gspo;
  int is_mode;
  float is_lo, is_hi;

  // loss of one token and its derivative wrt the probability ratio
  __device__ __forceinline__ void surrogate(float ratio, float a, float& loss, float& dratio,
                                            float& clipped) const {
    const float s1 = ratio * a;
    const float rc = fminf(fmaxf(ratio, lo), hi);
    const float in_clip = (ratio >= lo && ratio <= hi) ? 1.0f : 0.0f;  // clamp passes grad on [lo, hi]
    const float s2 = rc * a;
    // torch.min: gradient to the smaller operand, split evenly on ties
    const float w1 = s1 < s2 ? 1.0f : (s1 > s2 ? 0.0f : 0.5f);
    const float w2 = 1.0f - w1;
    float val = fminf(s1, s2);
    float dval = w1 * a + w2 * a * in_clip;  // d(min)/d(ratio)
    if (dual > 0.0f && a < 0.0f) {
      const float floor_v = dual * a;
      // torch.max(clip1, c*A): gradient to clip1 only where it is the larger one
      const float wk = val > floor_v ? 1.0f : (val < floor_v ? 0.0f : 0.5f);
      val = fmaxf(val, floor_v);
      dval *= wk;
    }
    if (s1 != s1 || s2 != s2) val = NAN;  // torch.min / torch.max propagate NaN, fminf does not
    loss = -val;
    dratio = -dval;
    clipped = s2 < s1 ? 1.0f : 0.0f;
  }

  // Inputs of one token, in the order the kernels hand them to eval() / grad(); a null pointer
  // marks an input this configuration does not read.
  static constexpr int kIn = 4;
  __device__ __forceinline__ const float* in(int j) const {
    if (j == 0) return lp;
    if (j == 1) return old;
    if (j == 2) return adv;
    return (is_mode != ORLHF_IS_NONE && !gspo) ? rollout : nullptr;
  }

  __device__ __forceinline__ float is_weight(int64_t b, float old_v, float roll_v) const {
    if (is_mode == ORLHF_IS_NONE || gspo) return 1.0f;
    const float w = expf(old_v - roll_v);
    if (is_mode == ORLHF_IS_TIS) return fminf(fmaxf(w, is_lo), is_hi);
    if (is_mode == ORLHF_IS_ICEPOP) return (w >= is_lo && w <= is_hi) ? w : 0.0f;
    return row_aux[b * 2] * w;  // seq-mask-tis: row keep flag times the unclamped token weight
  }

  // ratio and d(ratio)/d(lp) of the token's own log-prob (GSPO: handled by the caller)
  __device__ __forceinline__ void ppo_ratio(float raw, float& ratio, float& dr) const {
    const float c = fminf(fmaxf(raw, -20.0f), 20.0f);
    ratio = expf(c);
    dr = (raw >= -20.0f && raw <= 20.0f) ? ratio : 0.0f;
  }

  // v = {lp, old, adv, rollout} of the token
  __device__ __forceinline__ void eval(int64_t b, const float* v, float m, float* q) const {
    const float raw = v[0] - v[1];
    float ratio, dr;
    if (gspo) {
      ratio = row_aux[b * 2] * m;
    } else {
      ppo_ratio(raw, ratio, dr);
    }
    float loss, dratio, clipped;
    surrogate(ratio, v[2], loss, dratio, clipped);
    loss *= is_weight(b, v[1], v[3]);
    q[0] = loss * m;
    q[1] = m;
    q[2] = clipped * m;
    q[3] = -raw * m;
    q[4] = (is_mode != ORLHF_IS_NONE && !gspo) ? (v[3] - v[1]) * m : 0.0f;
  }

  // d(token loss)/d(lp) of a PPO token from its scalars (no memory access): used where the
  // log-prob has just been computed and is not in memory yet. `w` is the detached importance
  // weight (1 when no correction is applied).
  __device__ __forceinline__ float ppo_grad_of(float lp_v, float old_v, float adv_v, float w) const {
    float ratio, dr, loss, dratio, clipped;
    ppo_ratio(lp_v - old_v, ratio, dr);
    surrogate(ratio, adv_v, loss, dratio, clipped);
    return w * dratio * dr;
  }
  __device__ __forceinline__ float token_is_weight_of(float old_v, float roll_v) const {
    if (is_mode == ORLHF_IS_NONE) return 1.0f;
    const float w = expf(old_v - roll_v);
    if (is_mode == ORLHF_IS_TIS) return fminf(fmaxf(w, is_lo), is_hi);
    return (w >= is_lo && w <= is_hi) ? w : 0.0f;  // ICEPOP
  }

  // PPO: d(token loss)/d(lp).  GSPO: d(token loss)/d(ratio) * m (summed per row by the caller).
  __device__ __forceinline__ float grad(int64_t b, const float* v, float m) const {
    const float raw = v[0] - v[1];
    float ratio, dr;
    if (gspo) {
      ratio = row_aux[b * 2] * m;
      dr = m;
    } else {
      ppo_ratio(raw, ratio, dr);
    }
    float loss, dratio, clipped;
    surrogate(ratio, v[2], loss, dratio, clipped);
    return is_weight(b, v[1], v[3]) * dratio * dr;
  }
};

__device__ __forceinline__ void kl_value(int est, float d, float& v, float& dv) {
  if (est == ORLHF_KL_K1) {
    v = d;
    dv = 1.0f;
  } else if (est == ORLHF_KL_K2) {
    v = d * d / 2.0f;
    dv = d;
  } else {
    const float e = expf(-d);
    v = e - 1.0f + d;
    dv = 1.0f - e;
  }
  if (v == v) {  // NaN passes through untouched, like torch.clamp
    if (v < -10.0f || v > 10.0f) dv = 0.0f;  // clamp passes the gradient on the closed interval only
    v = fminf(fmaxf(v, -10.0f), 10.0f);
  }
}

}  // namespace orlhf
