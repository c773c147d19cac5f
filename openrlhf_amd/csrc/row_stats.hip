// Row-wise statistics kernels for gfx950 (forward only, the reference runs them without grad):
// the KL block of experience making (per-token KL estimate plus the per-sequence means the
// trainer logs) in one pass, and masked_normalize (per-row masked whitening). One workgroup per
// row, fp64 accumulation; the second and third walk of a row in masked_normalize hit the cache.
#include "token_terms.h"

namespace orlhf {

__device__ __forceinline__ void block_sum3(double& a, double& b, double& c, double (*lds)[kWavesPerBlock]) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    a += __shfl_xor(a, o, kWave);
    b += __shfl_xor(b, o, kWave);
    c += __shfl_xor(c, o, kWave);
  }
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[0][wave] = a, lds[1][wave] = b, lds[2][wave] = c;
  __syncthreads();
  a = b = c = 0.0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) a += lds[0][w], b += lds[1][w], c += lds[2][w];
  __syncthreads();
}

// kl[b,t] = clamp(estimator(lp - base), -10, 10); kl_mean[b] = sum(kl*m)/sum(m);
// diff_mean[b] = sum((lp - base)*m)/sum(m). enabled == 0: kl = 0 and both sums are of zeros.
template <int DT, int MASK_DT>
__global__ __launch_bounds__(kBlock) void kl_rows_kernel(const void* __restrict__ lp, const void* __restrict__ base,
                                                         const void* __restrict__ mask, Rows rows, int est,
                                                         int enabled, float* __restrict__ kl,
                                                         float* __restrict__ kl_mean,
                                                         float* __restrict__ diff_mean) {
  __shared__ double lds[3][kWavesPerBlock];
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t slot = blockIdx.x; slot < row_slots(rows.n_rows); slot += gridDim.x) {
    const int64_t b = row_of_slot(slot, slot, slot_b);
    if (b >= rows.n_rows) continue;
    const RowWalk rw = row_walk(rows, b);
    double sk = 0.0, sd = 0.0, sm = 0.0;
    auto token = [&](float x, float y, float m, float& v) {
      float d = 0.0f, dv;
      v = 0.0f;
      if (enabled) {
        d = x - y;
        kl_value(est, d, v, dv);
      }
      sk += (double)(v * m);
      sd += (double)(d * m);
      sm += (double)m;
    };
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          float x[4] = {0.0f, 0.0f, 0.0f, 0.0f}, y[4] = {0.0f, 0.0f, 0.0f, 0.0f}, m[4];
          if (enabled) {
            load_lp4<DT>(lp, i0, x);
            load_lp4<DT>(base, i0, y);
          }
          load_mask4<MASK_DT>(mask, i0, m);
          f32x4 v;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            float vk;
            token(x[k], y[k], m[k], vk);
            v[k] = vk;
          }
          if (kl != nullptr) *(f32x4e*)(kl + i0) = v;
        },
        [&](int64_t i) {
          float v;
          token(enabled ? load_lp<DT>(lp, i) : 0.0f, enabled ? load_lp<DT>(base, i) : 0.0f,
                load_mask<MASK_DT>(mask, i), v);
          if (kl != nullptr) kl[i] = v;
        });
    block_sum3(sk, sd, sm, lds);
    if (threadIdx.x == 0) {
      if (kl_mean != nullptr) kl_mean[b] = (float)(sk / sm);  // no epsilon: an empty row is NaN, as masked_mean
      if (diff_mean != nullptr) diff_mean[b] = (float)(sd / sm);
    }
  }
}

// out = (x - mean) * m * rsqrt(max(var, eps)), mean = sum(x*m)/max(sum(m), 1),
// var = sum(((x - mean)*m)^2)/max(sum(m), 1)
template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void masked_normalize_rows_kernel(const float* x,  // out may be x
                                                                       const void* __restrict__ mask, Rows rows,
                                                                       float eps, float* out) {
  __shared__ double lds[3][kWavesPerBlock];
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t slot = blockIdx.x; slot < row_slots(rows.n_rows); slot += gridDim.x) {
    const int64_t b = row_of_slot(slot, slot, slot_b);
    if (b >= rows.n_rows) continue;
    const RowWalk rw = row_walk(rows, b);
    double s = 0.0, c = 0.0, z = 0.0;
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          const f32x4 v = *(const f32x4e*)(x + i0);
          float m[4];
          load_mask4<MASK_DT>(mask, i0, m);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            s += (double)(v[k] * m[k]);
            c += (double)m[k];
          }
        },
        [&](int64_t i) {
          const float m = load_mask<MASK_DT>(mask, i);
          s += (double)(x[i] * m);
          c += (double)m;
        });
    block_sum3(s, c, z, lds);
    const double cnt = c < 1.0 ? 1.0 : c;
    const float mean = (float)(s / cnt);
    double v = 0.0, z1 = 0.0, z2 = 0.0;
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          const f32x4 xv = *(const f32x4e*)(x + i0);
          float m[4];
          load_mask4<MASK_DT>(mask, i0, m);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float e = (xv[k] - mean) * m[k];
            v += (double)(e * e);
          }
        },
        [&](int64_t i) {
          const float e = (x[i] - mean) * load_mask<MASK_DT>(mask, i);
          v += (double)(e * e);
        });
    block_sum3(v, z1, z2, lds);
    const float var = (float)(v / cnt);
    const float r = 1.0f / sqrtf(var != var ? var : fmaxf(var, eps));
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          const f32x4 xv = stream_load4(x + i0);
          float m[4];
          load_mask4<MASK_DT>(mask, i0, m);
          f32x4 o;
#pragma unroll
          for (int k = 0; k < 4; ++k) o[k] = (xv[k] - mean) * m[k] * r;
          *(f32x4e*)(out + i0) = o;
        },
        [&](int64_t i) { out[i] = (x[i] - mean) * load_mask<MASK_DT>(mask, i) * r; });
  }
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_kl_rows(const void* log_probs, const void* log_probs_base, int dtype, const void* mask,
                             int mask_dtype, int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                             int estimator, int enabled, float* kl, float* kl_mean, float* diff_mean,
                             orlhf_stream_t stream) {
  if (int rc = check_rows("kl_rows", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(estimator >= ORLHF_KL_K1 && estimator <= ORLHF_KL_K3, "kl_rows: unknown estimator %d", estimator);
  ORLHF_CHECK_ARG(dtype == ORLHF_F32 || dtype == ORLHF_BF16 || dtype == ORLHF_F16, "kl_rows: unknown dtype %d", dtype);
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(!enabled || n_cols == 0 || (log_probs != nullptr && log_probs_base != nullptr),
                  "kl_rows: log_probs / log_probs_base is NULL");
  const Rows rows{n_rows, n_cols, cu_seqlens};
  const dim3 grid(slot_grid(row_slots(n_rows), 65536)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_KL(M)                                                                                                  \
  do {                                                                                                               \
    if (dtype == ORLHF_F32)                                                                                          \
      hipLaunchKernelGGL((kl_rows_kernel<ORLHF_F32, M>), grid, block, 0, s, log_probs, log_probs_base, mask, rows,   \
                         estimator, enabled, kl, kl_mean, diff_mean);                                                \
    else if (dtype == ORLHF_BF16)                                                                                    \
      hipLaunchKernelGGL((kl_rows_kernel<ORLHF_BF16, M>), grid, block, 0, s, log_probs, log_probs_base, mask, rows,  \
                         estimator, enabled, kl, kl_mean, diff_mean);                                                \
    else                                                                                                             \
      hipLaunchKernelGGL((kl_rows_kernel<ORLHF_F16, M>), grid, block, 0, s, log_probs, log_probs_base, mask, rows,   \
                         estimator, enabled, kl, kl_mean, diff_mean);                                                \
  } while (0)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_KL)
#undef ORLHF_KL
  ORLHF_CHECK_LAUNCH("orlhf_kl_rows");
  return ORLHF_OK;
}

extern "C" int orlhf_masked_normalize_rows(const float* x, const void* mask, int mask_dtype, int64_t n_rows,
                                           int64_t n_cols, const int64_t* cu_seqlens, float eps, float* out,
                                           orlhf_stream_t stream) {
  if (int rc = check_rows("masked_normalize_rows", n_rows, n_cols, mask, mask_dtype)) return rc;
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(x != nullptr && out != nullptr, "masked_normalize_rows: NULL argument");
  const Rows rows{n_rows, n_cols, cu_seqlens};
  const dim3 grid(slot_grid(row_slots(n_rows), 65536)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_NORM(M) \
  hipLaunchKernelGGL(masked_normalize_rows_kernel<M>, grid, block, 0, s, x, mask, rows, eps, out)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_NORM)
#undef ORLHF_NORM
  ORLHF_CHECK_LAUNCH("orlhf_masked_normalize_rows");
  return ORLHF_OK;
}
