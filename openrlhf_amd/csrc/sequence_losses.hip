// Sequence-level kernels for gfx950 behind the preference trainers: per-sequence sums and means of
// per-token log-probs under the DPO loss mask (built on the fly from the attention mask and the
// prompt lengths), and the pairwise losses over [B] scalars (DPO sigmoid / IPO, reward-model
// pairwise and log-exp). One workgroup per sequence, fp64 accumulation, no atomics.
#include "common.h"

namespace orlhf {

// loss mask of column t of the shifted log-probs: attention_mask[b, t+1] != 0 and t+1 >= prompt_len[b]
template <int MASK_DT>
__device__ __forceinline__ float dpo_mask(const void* att, const int64_t* prompt_lens, int64_t b, int64_t t,
                                          int64_t att_cols) {
  const int64_t col = t + 1;
  if (prompt_lens != nullptr && col < prompt_lens[b]) return 0.0f;
  if (MASK_DT == ORLHF_MASK_NONE) return 1.0f;
  return load_mask<MASK_DT>(att, b * att_cols + col) != 0.0f ? 1.0f : 0.0f;
}

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void sequence_logps_fwd_kernel(const float* __restrict__ lp,
                                                                    const void* __restrict__ att,
                                                                    const int64_t* __restrict__ prompt_lens,
                                                                    int64_t n_rows, int64_t n_cols,
                                                                    float* __restrict__ sums,
                                                                    float* __restrict__ means,
                                                                    float* __restrict__ counts) {
  __shared__ double lds[kWavesPerBlock];
  const int slot_b = slot_bits(n_rows);
  for (int64_t slot = blockIdx.x; slot < row_slots(n_rows); slot += gridDim.x) {
    const int64_t b = row_of_slot(slot, slot, slot_b);
    if (b >= n_rows) continue;
    double s = 0.0, c = 0.0;
    // the mask sits one column to the right in rows one element longer: loads without alignment
    const Rows rows{n_rows, n_cols, nullptr};
    const RowWalk rw = row_walk(rows, b);
    auto token = [&](float x, int64_t t) {
      const float m = dpo_mask<MASK_DT>(att, prompt_lens, b, t, n_cols + 1);
      s += (double)(x * m);  // the reference multiplies by the mask (NaN * 0 stays NaN)
      c += (double)m;
    };
    const int64_t plen = prompt_lens != nullptr ? prompt_lens[b] : 0;
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          const f32x4 x = stream_load4(lp + i0);
          const int64_t t0 = i0 - b * n_cols;
          float a[4];
          load_mask4<MASK_DT>(att, b * (n_cols + 1) + t0 + 1, a);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float m = (t0 + k + 1 >= plen && a[k] != 0.0f) ? 1.0f : 0.0f;
            s += (double)(x[k] * m);
            c += (double)m;
          }
        },
        [&](int64_t i) { token(lp[i], i - b * n_cols); });
    s = block_sum(s, lds);
    c = block_sum(c, lds);
    if (threadIdx.x == 0) {
      const float sf = (float)s, cf = (float)c;
      if (sums != nullptr) sums[b] = sf;
      if (means != nullptr) means[b] = sf / cf;  // 0/0 = NaN for a sequence with no loss token, as torch
      if (counts != nullptr) counts[b] = cf;
    }
  }
}

constexpr int kSeqChunk = 4096;  // columns of one row per workgroup in the backward

// g[b,t] = m * (g_sum[b] + g_mean[b] / count[b])
template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void sequence_logps_bwd_kernel(const float* __restrict__ g_sums,
                                                                    const float* __restrict__ g_means,
                                                                    const void* __restrict__ att,
                                                                    const int64_t* __restrict__ prompt_lens,
                                                                    const float* __restrict__ counts,
                                                                    int64_t n_rows, int64_t n_cols,
                                                                    float* __restrict__ g) {
  const int64_t chunks = (n_cols + kSeqChunk - 1) / kSeqChunk;
  for (int64_t w = blockIdx.x; w < n_rows * chunks; w += gridDim.x) {
    const int64_t chunk = w / n_rows, b = w - chunk * n_rows, t0 = chunk * kSeqChunk;
    float up = g_sums != nullptr ? g_sums[b] : 0.0f;
    if (g_means != nullptr) up += g_means[b] / counts[b];
    const int64_t stop = t0 + kSeqChunk < n_cols ? t0 + kSeqChunk : n_cols;
    const int64_t plen = prompt_lens != nullptr ? prompt_lens[b] : 0;
    const int64_t groups = (stop - t0) / 4;  // four columns per lane: one mask load, one 16-byte store
#pragma unroll 2
    for (int64_t q = threadIdx.x; q < groups; q += kBlock) {
      const int64_t t = t0 + q * 4;
      float a[4];
      load_mask4<MASK_DT>(att, b * (n_cols + 1) + t + 1, a);
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = up * ((t + k + 1 >= plen && a[k] != 0.0f) ? 1.0f : 0.0f);
      *(f32x4e*)(g + b * n_cols + t) = o;
    }
    for (int64_t t = t0 + groups * 4 + threadIdx.x; t < stop; t += kBlock)
      g[b * n_cols + t] = up * dpo_mask<MASK_DT>(att, prompt_lens, b, t, n_cols + 1);
  }
}

// ---------------------------------------------------------------- pairwise losses over [n] scalars
__device__ __forceinline__ float log_sigmoid(float x) {  // min(x, 0) - log1p(exp(-|x|))
  return fminf(x, 0.0f) - log1pf(expf(-fabsf(x)));
}
__device__ __forceinline__ float sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

struct PairArgs {
  const float *a, *b, *c, *d;  // logit z = (a - b) - (c - d); c, d may be null (0)
  int64_t n;
  int kind;
  float beta, smooth;
};

__device__ __forceinline__ float pair_logit(const PairArgs& p, int64_t i) {
  const float pi = p.a[i] - p.b[i];
  if (p.c == nullptr && p.d == nullptr) return pi;
  const float ref = (p.c != nullptr ? p.c[i] : 0.0f) - (p.d != nullptr ? p.d[i] : 0.0f);
  return pi - ref;
}

// loss of one pair and its derivative with respect to the logit z
__device__ __forceinline__ void pair_term(const PairArgs& p, float z, float& loss, float& dz) {
  switch (p.kind) {
    case ORLHF_PAIR_DPO_SIGMOID: {
      const float x = p.beta * z;
      loss = -log_sigmoid(x) * (1.0f - p.smooth) - log_sigmoid(-x) * p.smooth;
      dz = p.beta * (-(1.0f - p.smooth) * sigmoid(-x) + p.smooth * sigmoid(x));
      break;
    }
    case ORLHF_PAIR_DPO_IPO: {
      const float e = z - 1.0f / (2.0f * p.beta);
      loss = e * e;
      dz = 2.0f * e;
      break;
    }
    case ORLHF_PAIR_LOGSIGMOID: {
      loss = -log_sigmoid(z);
      dz = -sigmoid(-z);
      break;
    }
    default: {  // ORLHF_PAIR_LOGEXP: log(1 + exp(-z)), the reference's unguarded form
      const float e = expf(-z);
      loss = logf(1.0f + e);
      dz = -(e / (1.0f + e));
      break;
    }
  }
}

__global__ __launch_bounds__(kBlock) void pair_loss_fwd_kernel(PairArgs p, float* __restrict__ loss_out,
                                                               float* __restrict__ chosen_rewards,
                                                               float* __restrict__ rejected_rewards) {
  __shared__ double lds[kWavesPerBlock];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < p.n; i += kBlock) {
    float loss, dz;
    pair_term(p, pair_logit(p, i), loss, dz);
    acc += (double)loss;
    if (chosen_rewards != nullptr) chosen_rewards[i] = p.beta * (p.a[i] - (p.c != nullptr ? p.c[i] : 0.0f));
    if (rejected_rewards != nullptr) rejected_rewards[i] = p.beta * (p.b[i] - (p.d != nullptr ? p.d[i] : 0.0f));
  }
  acc = block_sum(acc, lds);
  if (threadIdx.x == 0) loss_out[0] = (float)(acc / (double)p.n);  // mean of nothing = NaN, as torch
}

__global__ __launch_bounds__(kBlock) void pair_loss_bwd_kernel(PairArgs p, const float* __restrict__ g_out,
                                                               float* __restrict__ g_a, float* __restrict__ g_b) {
  const float up = g_out[0] / (float)p.n;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < p.n; i += (int64_t)gridDim.x * kBlock) {
    float loss, dz;
    pair_term(p, pair_logit(p, i), loss, dz);
    const float g = up * dz;
    if (g_a != nullptr) g_a[i] = g;
    if (g_b != nullptr) g_b[i] = -g;
  }
}

static int check_pair(const char* what, const float* a, const float* b, int64_t n, int kind, double beta,
                      double smooth) {
  if (n < 0) return fail(ORLHF_ERR_INVALID_ARG, "%s: n=%lld", what, (long long)n);
  if (n > 0 && (a == nullptr || b == nullptr)) return fail(ORLHF_ERR_INVALID_ARG, "%s: chosen/rejected is NULL", what);
  if (kind < ORLHF_PAIR_DPO_SIGMOID || kind > ORLHF_PAIR_LOGEXP)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: unknown pair loss kind %d", what, kind);
  if (!(beta == beta) || !(smooth == smooth)) return fail(ORLHF_ERR_INVALID_ARG, "%s: beta / label_smoothing is NaN", what);
  return ORLHF_OK;
}

static PairArgs pair_args(const float* a, const float* b, const float* c, const float* d, int64_t n, int kind,
                          double beta, double smooth) {
  PairArgs p;
  p.a = a, p.b = b, p.c = c, p.d = d, p.n = n, p.kind = kind;
  p.beta = (kind == ORLHF_PAIR_DPO_SIGMOID || kind == ORLHF_PAIR_DPO_IPO) ? (float)beta : 1.0f;
  p.smooth = (float)smooth;
  return p;
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_sequence_logps_fwd(const float* per_token_logps, const void* attention_mask, int mask_dtype,
                                        const int64_t* prompt_id_lens, int64_t n_rows, int64_t n_cols, float* sums,
                                        float* means, float* counts, orlhf_stream_t stream) {
  if (int rc = check_rows("sequence_logps_fwd", n_rows, n_cols, attention_mask, mask_dtype)) return rc;
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(per_token_logps != nullptr || n_cols == 0, "sequence_logps_fwd: per_token_logps is NULL");
  const dim3 grid(slot_grid(row_slots(n_rows), 65536)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_LAUNCH(M)                                                                                        \
  hipLaunchKernelGGL(sequence_logps_fwd_kernel<M>, grid, block, 0, s, per_token_logps, attention_mask, prompt_id_lens, \
                     n_rows, n_cols, sums, means, counts)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
  ORLHF_CHECK_LAUNCH("orlhf_sequence_logps_fwd");
  return ORLHF_OK;
}

extern "C" int orlhf_sequence_logps_bwd(const float* g_sums, const float* g_means, const void* attention_mask,
                                        int mask_dtype, const int64_t* prompt_id_lens, const float* counts,
                                        int64_t n_rows, int64_t n_cols, float* g_per_token, orlhf_stream_t stream) {
  if (int rc = check_rows("sequence_logps_bwd", n_rows, n_cols, attention_mask, mask_dtype)) return rc;
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(g_per_token != nullptr, "sequence_logps_bwd: g_per_token is NULL");
  ORLHF_CHECK_ARG(g_means == nullptr || counts != nullptr, "sequence_logps_bwd: g_means needs the forward's counts");
  const int64_t chunks = (n_cols + kSeqChunk - 1) / kSeqChunk;
  const dim3 grid((unsigned)(n_rows * chunks < 65536 ? n_rows * chunks : 65536)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_LAUNCH(M)                                                                                      \
  hipLaunchKernelGGL(sequence_logps_bwd_kernel<M>, grid, block, 0, s, g_sums, g_means, attention_mask, prompt_id_lens, \
                     counts, n_rows, n_cols, g_per_token)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
  ORLHF_CHECK_LAUNCH("orlhf_sequence_logps_bwd");
  return ORLHF_OK;
}

extern "C" int orlhf_pair_loss_fwd(const float* chosen, const float* rejected, const float* ref_chosen,
                                   const float* ref_rejected, int64_t n, int kind, double beta,
                                   double label_smoothing, float* loss, float* chosen_rewards,
                                   float* rejected_rewards, orlhf_stream_t stream) {
  if (int rc = check_pair("pair_loss_fwd", chosen, rejected, n, kind, beta, label_smoothing)) return rc;
  ORLHF_CHECK_ARG(loss != nullptr, "pair_loss_fwd: loss is NULL");
  const PairArgs p = pair_args(chosen, rejected, ref_chosen, ref_rejected, n, kind, beta, label_smoothing);
  hipLaunchKernelGGL(pair_loss_fwd_kernel, dim3(1), dim3(kBlock), 0, (hipStream_t)stream, p, loss, chosen_rewards,
                     rejected_rewards);
  ORLHF_CHECK_LAUNCH("orlhf_pair_loss_fwd");
  return ORLHF_OK;
}

extern "C" int orlhf_pair_loss_bwd(const float* g_out, const float* chosen, const float* rejected,
                                   const float* ref_chosen, const float* ref_rejected, int64_t n, int kind,
                                   double beta, double label_smoothing, float* g_chosen, float* g_rejected,
                                   orlhf_stream_t stream) {
  if (int rc = check_pair("pair_loss_bwd", chosen, rejected, n, kind, beta, label_smoothing)) return rc;
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(g_out != nullptr, "pair_loss_bwd: g_out is NULL");
  const PairArgs p = pair_args(chosen, rejected, ref_chosen, ref_rejected, n, kind, beta, label_smoothing);
  hipLaunchKernelGGL(pair_loss_bwd_kernel, dim3(flat_grid(n)), dim3(kBlock), 0, (hipStream_t)stream, p, g_out,
                     g_chosen, g_rejected);
  ORLHF_CHECK_LAUNCH("orlhf_pair_loss_bwd");
  return ORLHF_OK;
}
