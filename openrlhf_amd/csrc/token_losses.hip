// Per-token kernels for gfx950: approximate KL, masked token / sequence aggregation, the PPO
// (and GSPO) policy surrogate and the clipped value loss, each with its backward.
//
// Layout: a [n_rows, n_cols] problem is cut into chunks of 1024 to 8192 tokens of one row (8192
// on large batches); a workgroup walks one chunk in steps of 1024 tokens, four consecutive tokens
// per lane, and reduces the quantities it needs to one fp64 partial per (row, chunk), all
// quantities through the cross-lane steps together. A step is one 16-byte load per lane and array
// (and one load of four mask elements), wherever the row starts; only the lane that meets the
// row's end goes token by token (against 4-byte loads: PolicyLoss forward 206 -> 174 us,
// backward 286 -> 214 us on 67 M padded tokens). A fold kernel sums the chunks of each row, a
// single-workgroup kernel folds the rows in a fixed order and writes the scalars plus a per-row
// aggregation weight that the backward kernels multiply with. Chunks past the end of a short
// packed row return at once. No atomics anywhere: the result is bit-reproducible. All of these
// are HBM-bound streams of 4-17 bytes per token.
#include <atomic>

#include "token_terms.h"

namespace orlhf {

constexpr int kTokPerLane = 4;                // consecutive tokens per lane and step: one 16-byte load per array
constexpr int kSubChunk = kBlock * kTokPerLane;
constexpr int kMinChunk = kSubChunk;          // fewest tokens of one row per work item
constexpr int kMaxQ = 6;                      // quantities reduced per token
// Work items are (row, chunk) pairs numbered with the ROW varying fastest. Workgroups go to the
// eight XCDs round-robin by their index: numbered chunk-fastest, the chunks that hold tokens in a
// batch of short packed rows (chunk 0 and 1 of every row, say) would all land on the same two or
// four XCDs and the rest of the chip would only see the empty tail chunks. Within a chunk index
// the rows go through row_of_slot(), so that row lengths with a short period spread as well.
constexpr int64_t kMaxItemsGrid = 1 << 22;


// Chunks a row of up to n_cols tokens can span.
static inline int64_t chunks_of(const Rows& r) { return r.n_cols > 0 ? (r.n_cols + r.chunk - 1) / r.chunk : 1; }

// Rows of a chunked launch with the chunk length chosen for the problem size.
static Rows make_rows(int64_t n_rows, int64_t n_cols, const int64_t* cu) {
  // 8 steps per work item measured fastest on large batches (16 the same, 4: +8%, 2: +35%);
  // smaller problems get shorter chunks so that a thousand workgroups still exist.
  int steps = 8;
  while (steps > 1 && n_rows * ((n_cols + (int64_t)kSubChunk * steps - 1) / ((int64_t)kSubChunk * steps)) < 1024) steps /= 2;
  return Rows{n_rows, n_cols, cu, kSubChunk * steps};
}

struct NormArg {
  double dp_size, value;
  const float* dev;
};

static inline NormArg norm_arg(const orlhf_norm* n) {
  NormArg a;
  a.dp_size = n ? n->dp_size : 1.0;
  a.value = n ? n->norm_value : (double)NAN;
  a.dev = n ? n->norm_dev : nullptr;
  return a;
}

// ---------------------------------------------------------------- token functors
// Each functor evaluates one token: q[] are the quantities to reduce (already multiplied by the
// mask weight where the reference multiplies), and grad() is d(token loss)/d(input).

constexpr int kAggCounts = 100;  // internal finaliser mode: out = {sum(mask), #rows with sum(mask) > 0}

struct CountTok {  // loss normalisers: the mask alone
  static constexpr int kQ = 2, kIn = 0;
  __device__ __forceinline__ const float* in(int) const { return nullptr; }
  __device__ __forceinline__ void eval(int64_t, const float*, float m, float* q) const {
    q[0] = m;
    q[1] = m;
  }
};

struct AggTok {  // aggregate_loss / masked_mean: x*m and m
  static constexpr int kQ = 2, kIn = 1;
  const float* x;
  __device__ __forceinline__ const float* in(int) const { return x; }
  __device__ __forceinline__ void eval(int64_t, const float* v, float m, float* q) const {
    q[0] = v[0] * m;
    q[1] = m;
  }
};

struct ValueTok {  // quantities: masked loss, mask, masked value (for the mean value the trainer logs)
  static constexpr int kQ = 3, kIn = 3;
  const float *v, *old, *ret;
  int has_clip;
  float eps;
  __device__ __forceinline__ const float* in(int j) const {
    return j == 0 ? v : (j == 1 ? (has_clip ? old : nullptr) : ret);
  }
  // in = {value, old value, return}
  __device__ __forceinline__ void both(const float* in, float& loss, float& dv) const {
    const float x = in[0], r = in[2];
    const float e2 = x - r;
    const float b2 = e2 * e2;
    if (!has_clip) {
      loss = b2;
      dv = 2.0f * e2;
      return;
    }
    const float o = in[1];
    const float d = x - o;
    const float dc = fminf(fmaxf(d, -eps), eps);
    const float in_clip = (d >= -eps && d <= eps) ? 1.0f : 0.0f;
    const float e1 = (o + dc) - r;
    const float a2 = e1 * e1;
    // torch.max: gradient to the larger operand, split evenly on ties
    const float wa = a2 > b2 ? 1.0f : (a2 < b2 ? 0.0f : 0.5f);
    loss = fmaxf(a2, b2);
    if (a2 != a2 || b2 != b2) loss = NAN;
    dv = wa * 2.0f * e1 * in_clip + (1.0f - wa) * 2.0f * e2;
  }
  __device__ __forceinline__ void eval(int64_t, const float* in, float m, float* q) const {
    float loss, dv;
    both(in, loss, dv);
    q[0] = loss * m;
    q[1] = m;
    q[2] = in[0] * m;
  }
  __device__ __forceinline__ float grad(int64_t, const float* in, float) const {
    float loss, dv;
    both(in, loss, dv);
    return dv;
  }
};

struct RatioTok {  // row prepass: sum(lr*m), sum(m) with lr = a - b
  static constexpr int kQ = 2, kIn = 2;
  const float *a, *b;
  __device__ __forceinline__ const float* in(int j) const { return j == 0 ? a : b; }
  __device__ __forceinline__ void eval(int64_t, const float* v, float m, float* q) const {
    q[0] = (v[0] - v[1]) * m;
    q[1] = m;
  }
};

// PPO without importance correction and not GSPO: the common training configuration, with its
// branches settled at compile time (the general functor decides them per token at run time).
struct PlainPolicyTok {
  static constexpr int kQ = PolicyTok::kQ, kIn = 3;
  PolicyTok p;
  __device__ __forceinline__ const float* in(int j) const { return j == 0 ? p.lp : (j == 1 ? p.old : p.adv); }
  __device__ __forceinline__ void eval(int64_t, const float* v, float m, float* q) const {
    const float raw = v[0] - v[1];
    float ratio, dr, loss, dratio, clipped;
    p.ppo_ratio(raw, ratio, dr);
    p.surrogate(ratio, v[2], loss, dratio, clipped);
    q[0] = loss * m;
    q[1] = m;
    q[2] = clipped * m;
    q[3] = -raw * m;
    q[4] = 0.0f;
  }
  __device__ __forceinline__ float grad(int64_t, const float* v, float) const {
    float ratio, dr, loss, dratio, clipped;
    p.ppo_ratio(v[0] - v[1], ratio, dr);
    p.surrogate(ratio, v[2], loss, dratio, clipped);
    return dratio * dr;
  }
};

struct GspoGradTok {  // backward row sum: m * d(token loss)/d(ratio_t) * d(ratio_t)/d(s_b)
  static constexpr int kQ = 1, kIn = PolicyTok::kIn;
  PolicyTok p;
  __device__ __forceinline__ const float* in(int j) const { return p.in(j); }
  __device__ __forceinline__ void eval(int64_t b, const float* v, float m, float* q) const {
    q[0] = p.grad(b, v, m) * m;
  }
};

// ---------------------------------------------------------------- token loads
// A lane works on four consecutive tokens: one 16-byte load per input array and one load of the
// four mask elements.
template <typename Tok>
struct TokIn {
  static constexpr int kN = Tok::kIn > 0 ? Tok::kIn : 1;
};

template <typename Tok>
__device__ __forceinline__ void load_inputs(const Tok& tok, int64_t i, float* v) {
#pragma unroll
  for (int j = 0; j < Tok::kIn; ++j) {
    const float* p = tok.in(j);
    v[j] = p != nullptr ? p[i] : 0.0f;
  }
}

// i0: index of the first of four tokens
template <typename Tok>
__device__ __forceinline__ void load_inputs4(const Tok& tok, int64_t i0, float (*v)[TokIn<Tok>::kN]) {
#pragma unroll
  for (int j = 0; j < Tok::kIn; ++j) {
    const float* p = tok.in(j);
    f32x4 x = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p != nullptr) x = stream_load4(p + i0);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k][j] = x[k];
  }
}

// ---------------------------------------------------------------- stage 1: chunk partials
// STORE_GRAD: the aggregation weight of a token is known before the pass (token mean over a given
// count), so d(loss)/d(input 0) for a unit upstream gradient is written in the same pass:
// g_store[i] = w * m * tok.grad(...) with w = post_scale * dp_size / count, the float the finaliser
// puts into row_coef - the values rows_grad_kernel writes for g_out = 1, bit for bit.
template <int MASK_DT, typename Tok, bool STORE_GRAD>
__global__ __launch_bounds__(kBlock) void rows_partial_kernel(Rows rows, const void* __restrict__ mask,
                                                              Tok tok, double* __restrict__ partial,
                                                              int n_chunks, float* __restrict__ g_store,
                                                              NormArg norm, float post_scale) {
  constexpr int NQ = Tok::kQ;
  __shared__ double lds[NQ][kWavesPerBlock];
  float w = 0.0f;
  if (STORE_GRAD)
    w = (float)((double)post_scale * (norm.dp_size / (norm.dev != nullptr ? (double)norm.dev[0] : norm.value)));
  const int64_t slots = row_slots(rows.n_rows), items = slots * n_chunks;
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
    const int64_t chunk = item / slots, b = row_of_slot(item - chunk * slots, item, slot_b);  // rows vary fastest
    if (b >= rows.n_rows) continue;
    const RowWalk rw = row_walk(rows, b);
    const int64_t c0 = chunk * rows.chunk;
    double* out = partial + (b * n_chunks + chunk) * NQ;
    if (c0 >= rw.len) {  // a chunk past the end of a short (packed) row: nothing to read or reduce
      if (threadIdx.x < NQ) out[threadIdx.x] = 0.0;
      continue;
    }
    double acc[NQ];
#pragma unroll
    for (int i = 0; i < NQ; ++i) acc[i] = 0.0;
#pragma unroll 1
    for (int64_t s0 = c0; s0 < c0 + rows.chunk && s0 < rw.len; s0 += kSubChunk) {
      const int64_t t0 = s0 + (int64_t)threadIdx.x * kTokPerLane;
      if (t0 + kTokPerLane <= rw.len) {  // this lane's four tokens lie in the row
        const int64_t i0 = rw.base + t0;
        float v[kTokPerLane][TokIn<Tok>::kN], m[kTokPerLane], q[kTokPerLane][NQ];
        load_inputs4(tok, i0, v);
        load_mask4<MASK_DT>(mask, i0, m);
#pragma unroll
        for (int k = 0; k < kTokPerLane; ++k) tok.eval(b, v[k], m[k], q[k]);
#pragma unroll
        for (int k = 0; k < kTokPerLane; ++k) {
#pragma unroll
          for (int i = 0; i < NQ; ++i) acc[i] += (double)q[k][i];
        }
        if constexpr (STORE_GRAD) {
          f32x4 go;
#pragma unroll
          for (int k = 0; k < kTokPerLane; ++k) go[k] = w * m[k] * tok.grad(b, v[k], m[k]);
          *(f32x4e*)(g_store + i0) = go;
        }
      } else {  // the lane that meets the row's end, and the lanes past it
#pragma unroll
        for (int k = 0; k < kTokPerLane; ++k) {
          if (t0 + k < rw.len) {
            const float m = load_mask<MASK_DT>(mask, rw.base + t0 + k);
            float v[TokIn<Tok>::kN], q[NQ];
            load_inputs(tok, rw.base + t0 + k, v);
            tok.eval(b, v, m, q);
#pragma unroll
            for (int i = 0; i < NQ; ++i) acc[i] += (double)q[i];
            if constexpr (STORE_GRAD) g_store[rw.base + t0 + k] = w * m * tok.grad(b, v, m);
          }
        }
      }
    }
    // all quantities through the wave shuffles together (independent chains), one barrier
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) acc[i] += __shfl_xor(acc[i], o, kWave);
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) lds[i][wave] = acc[i];
    }
    __syncthreads();
    if (threadIdx.x < NQ) {
      double r = 0.0;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) r += lds[threadIdx.x][w];
      out[threadIdx.x] = r;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- stage 2: rows -> scalars
// Quantity 0 is the loss numerator, quantity 1 the mask weight; quantities 2.. are numerators of
// plain masked means. out[0] = post_scale * aggregate(q0); out[k-1] = sum(qk)/sum(q1), k >= 2.
// row_coef[b] = post_scale * d(aggregate)/d(row b's masked token sum).
constexpr int kFinalRows = 8;  // rows per lane whose loads the finaliser issues together

template <int NQ>
__global__ __launch_bounds__(kBlock) void rows_final_kernel(int64_t n_rows,
                                                            const double* __restrict__ row_total, int mode,
                                                            NormArg norm, float post_scale, int n_out,
                                                            float* __restrict__ out,
                                                            float* __restrict__ row_coef) {
  __shared__ double lds[NQ + 2][kWavesPerBlock];
  double tot[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) tot[i] = 0.0;
  double seq_sum = 0.0, seq_cnt = 0.0;
  // One workgroup walks all rows: the loads of kFinalRows rows per lane are issued together, or
  // the walk is a chain of load latencies (18 us for 4096 rows with one row at a time).
  for (int64_t b0 = threadIdx.x; b0 < n_rows; b0 += (int64_t)kFinalRows * kBlock) {
    double batch[kFinalRows][NQ];
#pragma unroll
    for (int u = 0; u < kFinalRows; ++u) {
      const int64_t b = b0 + (int64_t)u * kBlock;
#pragma unroll
      for (int i = 0; i < NQ; ++i) batch[u][i] = b < n_rows ? row_total[b * NQ + i] : 0.0;
    }
#pragma unroll
    for (int u = 0; u < kFinalRows; ++u) {
      const int64_t b = b0 + (int64_t)u * kBlock;
      if (b >= n_rows) break;
      const double* rq = batch[u];
#pragma unroll
      for (int i = 0; i < NQ; ++i) tot[i] += rq[i];
      if (mode == ORLHF_AGG_SEQ_MEAN || mode == ORLHF_AGG_SEQ_MEAN_TOKEN_SUM || mode == kAggCounts) {
        if (rq[1] > 0.0) {
          seq_sum += mode == ORLHF_AGG_SEQ_MEAN_TOKEN_SUM ? rq[0] : rq[0] / (rq[1] + 1e-8);
          seq_cnt += 1.0;
        } else if (rq[0] != rq[0]) {
          seq_sum += rq[0];  // NaN * 0 stays NaN in the reference
        }
      } else if (mode == ORLHF_AGG_ROW_MEAN) {
        out[b] = (float)(rq[0] / rq[1]);
      }
      if (row_coef != nullptr) row_coef[b] = (float)rq[1];  // finished below
    }
  }
  if (mode == ORLHF_AGG_ROW_MEAN) {
    if (row_coef != nullptr) {
      __syncthreads();
      for (int64_t b = threadIdx.x; b < n_rows; b += kBlock) row_coef[b] = 1.0f / row_coef[b];
    }
    return;
  }
  // every sum through the cross-lane steps together, one LDS exchange for all of them
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
#pragma unroll
    for (int i = 0; i < NQ; ++i) tot[i] += __shfl_xor(tot[i], o, kWave);
    seq_sum += __shfl_xor(seq_sum, o, kWave);
    seq_cnt += __shfl_xor(seq_cnt, o, kWave);
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    const int wave = threadIdx.x / kWave;
#pragma unroll
    for (int i = 0; i < NQ; ++i) lds[i][wave] = tot[i];
    lds[NQ][wave] = seq_sum;
    lds[NQ + 1][wave] = seq_cnt;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    tot[i] = 0.0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) tot[i] += lds[i][w];
  }
  seq_sum = seq_cnt = 0.0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    seq_sum += lds[NQ][w];
    seq_cnt += lds[NQ + 1][w];
  }

  if (mode == kAggCounts) {
    if (threadIdx.x == 0) {
      out[0] = (float)tot[1];
      out[1] = (float)seq_cnt;
    }
    return;
  }
  const bool given = norm.dev != nullptr || norm.value == norm.value;
  const double denom_given = norm.dev != nullptr ? (double)norm.dev[0] : norm.value;
  double scale;  // d(loss)/d(numerator)
  double loss;
  if (mode == ORLHF_AGG_TOKEN_MEAN) {
    scale = given ? norm.dp_size / denom_given : 1.0 / tot[1];
    loss = given ? tot[0] / denom_given * norm.dp_size : tot[0] / tot[1];
  } else {
    scale = given ? norm.dp_size / denom_given : 1.0 / seq_cnt;
    loss = given ? seq_sum / denom_given * norm.dp_size : seq_sum / seq_cnt;
  }
  if (threadIdx.x == 0) {
    out[0] = (float)((double)post_scale * loss);
    for (int i = 2; i < NQ && i - 1 < n_out; ++i) out[i - 1] = (float)(tot[i] / tot[1]);
  }
  if (row_coef != nullptr) {
    for (int64_t b0 = threadIdx.x; b0 < n_rows; b0 += (int64_t)kFinalRows * kBlock) {
      float cnt_f[kFinalRows];
#pragma unroll
      for (int u = 0; u < kFinalRows; ++u) {
        const int64_t b = b0 + (int64_t)u * kBlock;
        cnt_f[u] = b < n_rows ? row_coef[b] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < kFinalRows; ++u) {
        const int64_t b = b0 + (int64_t)u * kBlock;
        if (b >= n_rows) break;
        const double cnt = (double)cnt_f[u];
        double c;
        if (mode == ORLHF_AGG_TOKEN_MEAN)
          c = scale;
        else if (mode == ORLHF_AGG_SEQ_MEAN_TOKEN_SUM)
          c = cnt > 0.0 ? scale : 0.0;
        else
          c = cnt > 0.0 ? scale / (cnt + 1e-8) : 0.0;
        row_coef[b] = (float)((double)post_scale * c);
      }
    }
  }
}

// Stage 1b: fold the chunk partials of every row into one entry per row, one lane per row, so
// that the single-workgroup finaliser reads n_rows entries instead of n_rows * n_chunks.
template <int NQ>
__global__ __launch_bounds__(kBlock) void rows_fold_kernel(int64_t n_rows, int n_chunks,
                                                           const double* __restrict__ partial,
                                                           double* __restrict__ row_total) {
  for (int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x; b < n_rows; b += (int64_t)gridDim.x * kBlock) {
    double rq[NQ];
#pragma unroll
    for (int i = 0; i < NQ; ++i) rq[i] = 0.0;
    for (int c = 0; c < n_chunks; ++c) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) rq[i] += partial[(b * n_chunks + c) * NQ + i];
    }
#pragma unroll
    for (int i = 0; i < NQ; ++i) row_total[b * NQ + i] = rq[i];
  }
}

// Row prepass results for GSPO (kind 0) and seq-mask-TIS (kind 1): row_aux[b] = {value, 1/max(cnt,1)}.
__global__ __launch_bounds__(kBlock) void row_aux_kernel(int64_t n_rows, int n_chunks,
                                                         const double* __restrict__ partial, int kind,
                                                         float is_lo, float is_hi,
                                                         float* __restrict__ row_aux) {
  for (int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x; b < n_rows; b += (int64_t)gridDim.x * kBlock) {
    double s = 0.0, cnt = 0.0;
    for (int c = 0; c < n_chunks; ++c) {
      s += partial[(b * n_chunks + c) * 2];
      cnt += partial[(b * n_chunks + c) * 2 + 1];
    }
    const float inv = (float)(1.0 / (cnt > 1.0 ? cnt : 1.0));
    float v;
    if (kind == 0) {
      v = expf((float)(s / (cnt > 1.0 ? cnt : 1.0)));  // exp(sum(lr*m) / clamp(sum(m), 1))
    } else {
      const float w = expf((float)(s / cnt));  // exp(masked_mean): NaN for an empty row -> dropped
      v = (w >= is_lo && w <= is_hi) ? 1.0f : 0.0f;
    }
    row_aux[b * 2] = v;
    row_aux[b * 2 + 1] = inv;
  }
}

// ---------------------------------------------------------------- backward, elementwise
// g[b,t] = g_out * row_coef[b] * m * tok.grad(...)
template <int MASK_DT, typename Tok>
__global__ __launch_bounds__(kBlock) void rows_grad_kernel(Rows rows, const void* __restrict__ mask, Tok tok,
                                                           const float* __restrict__ g_out, int g_per_row,
                                                           const float* __restrict__ row_coef,
                                                           float* __restrict__ g, int n_chunks) {
  const int64_t slots = row_slots(rows.n_rows), items = slots * n_chunks;
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
    const int64_t chunk = item / slots, b = row_of_slot(item - chunk * slots, item, slot_b);  // rows vary fastest
    if (b >= rows.n_rows) continue;
    const RowWalk rw = row_walk(rows, b);
    const int64_t c0 = chunk * rows.chunk;
    if (c0 >= rw.len) continue;
    const float w = (g_per_row ? g_out[b] : g_out[0]) * row_coef[b];
#pragma unroll 1
    for (int64_t s0 = c0; s0 < c0 + rows.chunk && s0 < rw.len; s0 += kSubChunk) {
      const int64_t t0 = s0 + (int64_t)threadIdx.x * kTokPerLane;
      if (t0 + kTokPerLane <= rw.len) {
        const int64_t i0 = rw.base + t0;
        float v[kTokPerLane][TokIn<Tok>::kN], m[kTokPerLane];
        load_inputs4(tok, i0, v);
        load_mask4<MASK_DT>(mask, i0, m);
        f32x4 out;
#pragma unroll
        for (int k = 0; k < kTokPerLane; ++k) out[k] = w * m[k] * tok.grad(b, v[k], m[k]);
        *(f32x4e*)(g + i0) = out;
      } else {
#pragma unroll
        for (int k = 0; k < kTokPerLane; ++k) {
          if (t0 + k < rw.len) {
            const float m = load_mask<MASK_DT>(mask, rw.base + t0 + k);
            float v[TokIn<Tok>::kN];
            load_inputs(tok, rw.base + t0 + k, v);
            g[rw.base + t0 + k] = w * m * tok.grad(b, v, m);
          }
        }
      }
    }
  }
}

struct UnitGrad {  // aggregate backward: d(x*m)/dx / m = 1
  static constexpr int kIn = 0;
  __device__ __forceinline__ const float* in(int) const { return nullptr; }
  __device__ __forceinline__ float grad(int64_t, const float*, float) const { return 1.0f; }
};

// GSPO backward: g[b,t] = g_out * row_coef[b] * rowsum_b * s_b * m / max(cnt_b, 1)
template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void gspo_grad_kernel(Rows rows, const void* __restrict__ mask,
                                                           const double* __restrict__ partial, int n_chunks,
                                                           const float* __restrict__ g_out,
                                                           const float* __restrict__ row_coef,
                                                           const float* __restrict__ row_aux,
                                                           float* __restrict__ g) {
  const int64_t slots = row_slots(rows.n_rows), items = slots * n_chunks;
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
    const int64_t chunk = item / slots, b = row_of_slot(item - chunk * slots, item, slot_b);  // rows vary fastest
    if (b >= rows.n_rows) continue;
    int64_t start, len;
    row_span(rows, b, start, len);
    const int64_t c0 = chunk * rows.chunk;
    if (c0 >= len) continue;
    double rs = 0.0;
    for (int c = 0; c < n_chunks; ++c) rs += partial[b * n_chunks + c];
    const float w = g_out[0] * row_coef[b] * (float)rs * row_aux[b * 2] * row_aux[b * 2 + 1];
    for (int64_t t = c0 + threadIdx.x; t < c0 + rows.chunk && t < len; t += kBlock)
      g[start + t] = w * load_mask<MASK_DT>(mask, start + t);
  }
}

// ---------------------------------------------------------------- approximate KL (flat)
template <int DT>
__global__ __launch_bounds__(kBlock) void approx_kl_fwd_kernel(const void* __restrict__ lp,
                                                               const void* __restrict__ base, int64_t n, int est,
                                                               float* __restrict__ out) {
  const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x, stride = (int64_t)gridDim.x * kBlock;
  const int64_t groups = n / 4;
#pragma unroll 2
  for (int64_t g = first; g < groups; g += stride) {
    float x[4], y[4];
    load_lp4<DT>(lp, g * 4, x);
    load_lp4<DT>(base, g * 4, y);
    f32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float v, dv;
      kl_value(est, x[k] - y[k], v, dv);
      o[k] = v;
    }
    *(f32x4e*)(out + g * 4) = o;
  }
  for (int64_t i = groups * 4 + first; i < n; i += stride) {
    float v, dv;
    kl_value(est, load_lp<DT>(lp, i) - load_lp<DT>(base, i), v, dv);
    out[i] = v;
  }
}

template <int DT>
__global__ __launch_bounds__(kBlock) void approx_kl_bwd_kernel(const void* __restrict__ lp,
                                                               const void* __restrict__ base, int64_t n, int est,
                                                               const float* __restrict__ g_out,
                                                               float* __restrict__ g_lp, float* __restrict__ g_base) {
  const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x, stride = (int64_t)gridDim.x * kBlock;
  const int64_t groups = n / 4;
#pragma unroll 2
  for (int64_t g = first; g < groups; g += stride) {
    float x[4], y[4];
    load_lp4<DT>(lp, g * 4, x);
    load_lp4<DT>(base, g * 4, y);
    const f32x4 up = stream_load4(g_out + g * 4);
    f32x4 o, neg;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float v, dv;
      kl_value(est, x[k] - y[k], v, dv);
      o[k] = up[k] * dv;
      neg[k] = -o[k];
    }
    if (g_lp != nullptr) *(f32x4e*)(g_lp + g * 4) = o;
    if (g_base != nullptr) *(f32x4e*)(g_base + g * 4) = neg;
  }
  for (int64_t i = groups * 4 + first; i < n; i += stride) {
    float v, dv;
    kl_value(est, load_lp<DT>(lp, i) - load_lp<DT>(base, i), v, dv);
    const float g = g_out[i] * dv;
    if (g_lp != nullptr) g_lp[i] = g;
    if (g_base != nullptr) g_base[i] = -g;
  }
}

// ---------------------------------------------------------------- host helpers
static inline dim3 row_grid(const Rows& rows) {
  return dim3(slot_grid(row_slots(rows.n_rows) * chunks_of(rows), kMaxItemsGrid));
}

template <typename Tok>
static void launch_partial(int mask_dt, Rows rows, const void* mask, const Tok& tok, double* partial,
                           int n_chunks, hipStream_t s) {
  const dim3 grid = row_grid(rows), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                      \
  hipLaunchKernelGGL((rows_partial_kernel<M, Tok, false>), grid, block, 0, s, rows, mask, tok, partial, n_chunks, \
                     (float*)nullptr, NormArg{1.0, 1.0, nullptr}, 1.0f)
  ORLHF_FOR_MASK_DTYPE(mask_dt, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
}

// Chunk partials plus the gradient for a unit upstream gradient in the same pass (token mean over a
// given count only: see rows_partial_kernel). g_store == nullptr is the plain launch.
template <typename Tok>
static void launch_partial_grad(int mask_dt, Rows rows, const void* mask, const Tok& tok, double* partial,
                                int n_chunks, float* g_store, const NormArg& norm, float post_scale, hipStream_t s) {
  if (g_store == nullptr) {
    launch_partial(mask_dt, rows, mask, tok, partial, n_chunks, s);
    return;
  }
  const dim3 grid = row_grid(rows), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                     \
  hipLaunchKernelGGL((rows_partial_kernel<M, Tok, true>), grid, block, 0, s, rows, mask, tok, partial, n_chunks, \
                     g_store, norm, post_scale)
  ORLHF_FOR_MASK_DTYPE(mask_dt, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
}

template <typename Tok>
static void launch_grad(int mask_dt, Rows rows, const void* mask, const Tok& tok, const float* g_out,
                        int g_per_row, const float* row_coef, float* g, hipStream_t s) {
  const dim3 grid = row_grid(rows), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                    \
  hipLaunchKernelGGL((rows_grad_kernel<M, Tok>), grid, block, 0, s, rows, mask, tok, g_out, g_per_row, row_coef, g, \
                     (int)chunks_of(rows))
  ORLHF_FOR_MASK_DTYPE(mask_dt, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
}


// Folds chunk partials per row (when there is more than one chunk) and runs the finaliser.
template <int NQ>
static void launch_final(int64_t n_rows, int n_chunks, double* partial, int mode, const NormArg& norm,
                         float post_scale, int n_out, float* out, float* row_coef, hipStream_t s) {
  const double* src = partial;  // one chunk per row: the partials are the row totals
  if (n_chunks > 1 && n_rows > 0) {
    double* row_total = partial + n_rows * (int64_t)n_chunks * NQ;
    hipLaunchKernelGGL(rows_fold_kernel<NQ>, dim3(flat_grid(n_rows, 4096)), dim3(kBlock), 0, s, n_rows, n_chunks,
                       partial, row_total);
    src = row_total;
  }
  hipLaunchKernelGGL(rows_final_kernel<NQ>, dim3(1), dim3(kBlock), 0, s, n_rows, src, mode, norm, post_scale, n_out,
                     out, row_coef);
}

static PolicyTok policy_tok(const float* lp, const float* old, const float* adv, const float* rollout,
                            const float* row_aux, const orlhf_policy_params* p) {
  PolicyTok t;
  t.lp = lp;
  t.old = old;
  t.adv = adv;
  t.rollout = rollout;
  t.row_aux = row_aux;
  t.lo = 1.0f - p->clip_eps_low;
  t.hi = 1.0f + p->clip_eps_high;
  t.dual = p->dual_clip;
  t.gspo = p->policy_type == ORLHF_POLICY_GSPO;
  t.is_mode = p->is_correction;
  t.is_lo = p->is_low;
  t.is_hi = p->is_high;
  return t;
}

static int check_policy(const char* what, const orlhf_policy_params* p, const float* rollout) {
  if (p == nullptr) return fail(ORLHF_ERR_INVALID_ARG, "%s: params is NULL", what);
  if (p->policy_type != ORLHF_POLICY_PPO && p->policy_type != ORLHF_POLICY_GSPO)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: unknown policy_type %d", what, p->policy_type);
  if (p->is_correction < ORLHF_IS_NONE || p->is_correction > ORLHF_IS_SEQ_MASK_TIS)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: unknown is_correction %d", what, p->is_correction);
  if (p->is_correction != ORLHF_IS_NONE && rollout == nullptr)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: importance correction needs rollout_log_probs", what);
  if (p->dual_clip > 0.0f && !(p->dual_clip > 1.0f))
    return fail(ORLHF_ERR_INVALID_ARG, "%s: dual_clip must be > 1.0, got %g", what, (double)p->dual_clip);
  return ORLHF_OK;
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int64_t orlhf_token_workspace_bytes(int64_t n_rows, int64_t n_cols) {
  if (n_rows < 0 || n_cols < 0) return 0;
  // chunk partials, then one folded entry per row
  const int64_t chunks = n_cols > 0 ? (n_cols + kMinChunk - 1) / kMinChunk : 1;  // the most chunks_of() returns
  return (n_rows > 0 ? n_rows : 1) * (chunks + 1) * kMaxQ * (int64_t)sizeof(double) + 256;
}

extern "C" int orlhf_approx_kl_fwd(const void* log_probs, const void* log_probs_base, int dtype, int64_t n,
                                   int estimator, float* out, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0, "approx_kl_fwd: n=%lld", (long long)n);
  ORLHF_CHECK_ARG(estimator >= ORLHF_KL_K1 && estimator <= ORLHF_KL_K3, "approx_kl_fwd: unknown estimator %d", estimator);
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(log_probs && log_probs_base && out, "approx_kl_fwd: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_grid((n + 3) / 4)), block(kBlock);
  switch (dtype) {
    case ORLHF_F32: hipLaunchKernelGGL(approx_kl_fwd_kernel<ORLHF_F32>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, out); break;
    case ORLHF_BF16: hipLaunchKernelGGL(approx_kl_fwd_kernel<ORLHF_BF16>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, out); break;
    case ORLHF_F16: hipLaunchKernelGGL(approx_kl_fwd_kernel<ORLHF_F16>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, out); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "approx_kl_fwd: unknown dtype %d", dtype);
  }
  ORLHF_CHECK_LAUNCH("orlhf_approx_kl_fwd");
  return ORLHF_OK;
}

extern "C" int orlhf_approx_kl_bwd(const void* log_probs, const void* log_probs_base, int dtype, int64_t n,
                                   int estimator, const float* g_out, float* g_lp, float* g_base,
                                   orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0, "approx_kl_bwd: n=%lld", (long long)n);
  ORLHF_CHECK_ARG(estimator >= ORLHF_KL_K1 && estimator <= ORLHF_KL_K3, "approx_kl_bwd: unknown estimator %d", estimator);
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(log_probs && log_probs_base && g_out && (g_lp || g_base), "approx_kl_bwd: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(flat_grid((n + 3) / 4)), block(kBlock);
  switch (dtype) {
    case ORLHF_F32: hipLaunchKernelGGL(approx_kl_bwd_kernel<ORLHF_F32>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, g_out, g_lp, g_base); break;
    case ORLHF_BF16: hipLaunchKernelGGL(approx_kl_bwd_kernel<ORLHF_BF16>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, g_out, g_lp, g_base); break;
    case ORLHF_F16: hipLaunchKernelGGL(approx_kl_bwd_kernel<ORLHF_F16>, grid, block, 0, s, log_probs, log_probs_base, n, estimator, g_out, g_lp, g_base); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "approx_kl_bwd: unknown dtype %d", dtype);
  }
  ORLHF_CHECK_LAUNCH("orlhf_approx_kl_bwd");
  return ORLHF_OK;
}

extern "C" int orlhf_masked_aggregate_fwd(const float* x, const void* mask, int mask_dtype, int64_t n_rows,
                                          int64_t n_cols, const int64_t* cu_seqlens, int mode,
                                          const orlhf_norm* norm, void* workspace, float* out,
                                          float* row_coef, orlhf_stream_t stream) {
  if (int rc = check_rows("masked_aggregate_fwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mode >= ORLHF_AGG_TOKEN_MEAN && mode <= ORLHF_AGG_SEQ_MEAN_TOKEN_SUM, "masked_aggregate_fwd: unknown mode %d", mode);
  ORLHF_CHECK_ARG(out != nullptr && workspace != nullptr, "masked_aggregate_fwd: NULL out / workspace");
  ORLHF_CHECK_ARG(x != nullptr || n_rows * n_cols == 0, "masked_aggregate_fwd: x is NULL");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  if (n_rows > 0) {
    AggTok tok{x};
    launch_partial(mask_dtype, rows, mask, tok, partial, n_chunks, s);
    ORLHF_CHECK_LAUNCH("orlhf_masked_aggregate_fwd(partial)");
  }
  launch_final<2>(n_rows, n_chunks, partial, mode, norm_arg(norm), 1.0f, 1, out, row_coef, s);
  ORLHF_CHECK_LAUNCH("orlhf_masked_aggregate_fwd(final)");
  return ORLHF_OK;
}

extern "C" int orlhf_mask_counts(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                                 const int64_t* cu_seqlens, void* workspace, float* out2, orlhf_stream_t stream) {
  if (int rc = check_rows("mask_counts", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(out2 != nullptr && workspace != nullptr, "mask_counts: NULL out2 / workspace");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  if (n_rows > 0) {
    launch_partial(mask_dtype, rows, mask, CountTok{}, partial, n_chunks, s);
    ORLHF_CHECK_LAUNCH("orlhf_mask_counts(partial)");
  }
  NormArg none{1.0, (double)NAN, nullptr};
  launch_final<2>(n_rows, n_chunks, partial, kAggCounts, none, 1.0f, 2, out2, nullptr, s);
  ORLHF_CHECK_LAUNCH("orlhf_mask_counts(final)");
  return ORLHF_OK;
}

extern "C" int orlhf_mask_row_coef(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols, int mode,
                                   const orlhf_norm* norm, void* workspace, float* row_coef, orlhf_stream_t stream) {
  if (int rc = check_rows("mask_row_coef", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mode == ORLHF_AGG_TOKEN_MEAN || mode == ORLHF_AGG_SEQ_MEAN || mode == ORLHF_AGG_SEQ_MEAN_TOKEN_SUM,
                  "mask_row_coef: mode %d has no scalar aggregate", mode);
  ORLHF_CHECK_ARG(row_coef != nullptr && workspace != nullptr, "mask_row_coef: NULL row_coef / workspace");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, nullptr);
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  if (n_rows > 0) {
    launch_partial(mask_dtype, rows, mask, CountTok{}, partial, n_chunks, s);
    ORLHF_CHECK_LAUNCH("orlhf_mask_row_coef(partial)");
  }
  // the aggregate of the mask itself is of no interest: it goes to the spare tail of the workspace
  float* unused = (float*)((char*)workspace + orlhf_token_workspace_bytes(n_rows, n_cols) - 256);
  launch_final<2>(n_rows, n_chunks, partial, mode, norm_arg(norm), 1.0f, 1, unused, row_coef, s);
  ORLHF_CHECK_LAUNCH("orlhf_mask_row_coef(final)");
  return ORLHF_OK;
}

extern "C" int orlhf_masked_aggregate_bwd(const float* g_out, const void* mask, int mask_dtype, int64_t n_rows,
                                          int64_t n_cols, const int64_t* cu_seqlens, int mode,
                                          const float* row_coef, float* g_x, orlhf_stream_t stream) {
  if (int rc = check_rows("masked_aggregate_bwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mode >= ORLHF_AGG_TOKEN_MEAN && mode <= ORLHF_AGG_SEQ_MEAN_TOKEN_SUM, "masked_aggregate_bwd: unknown mode %d", mode);
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(g_out && row_coef && g_x, "masked_aggregate_bwd: NULL pointer");
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  launch_grad(mask_dtype, rows, mask, UnitGrad{}, g_out, mode == ORLHF_AGG_ROW_MEAN, row_coef, g_x, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_masked_aggregate_bwd");
  return ORLHF_OK;
}

// The weight of a token in the loss is known before the pass: token mean over a count the caller gives.
static bool norm_given(const orlhf_norm* n) { return n != nullptr && (n->norm_dev != nullptr || n->norm_value == n->norm_value); }

static int policy_loss_fwd_impl(const float* log_probs, const float* old_log_probs, const float* advantages,
                                const void* mask, int mask_dtype, const float* rollout_log_probs,
                                int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                                const orlhf_policy_params* params, void* workspace, float* out4,
                                float* row_coef, float* row_aux, float* g_store, orlhf_stream_t stream) {
  if (int rc = check_rows("policy_loss_fwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  if (int rc = check_policy("policy_loss_fwd", params, rollout_log_probs)) return rc;
  ORLHF_CHECK_ARG(out4 && workspace && row_aux, "policy_loss_fwd: NULL out4 / workspace / row_aux");
  ORLHF_CHECK_ARG((log_probs && old_log_probs && advantages) || n_rows * n_cols == 0, "policy_loss_fwd: NULL input");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  const bool gspo = params->policy_type == ORLHF_POLICY_GSPO;
  const bool use_is = params->is_correction != ORLHF_IS_NONE;
  if (n_rows > 0 && (gspo || params->is_correction == ORLHF_IS_SEQ_MASK_TIS)) {
    RatioTok pre;
    if (gspo) {
      pre.a = log_probs;
      pre.b = use_is ? rollout_log_probs : old_log_probs;
    } else {
      pre.a = old_log_probs;
      pre.b = rollout_log_probs;
    }
    launch_partial(mask_dtype, rows, mask, pre, partial, n_chunks, s);
    ORLHF_CHECK_LAUNCH("orlhf_policy_loss_fwd(prepass)");
    hipLaunchKernelGGL(row_aux_kernel, dim3(flat_grid(n_rows)), dim3(kBlock), 0, s, n_rows, n_chunks, partial,
                       gspo ? 0 : 1, params->is_low, params->is_high, row_aux);
    ORLHF_CHECK_LAUNCH("orlhf_policy_loss_fwd(row_aux)");
  }
  if (n_rows > 0) {
    PolicyTok tok = policy_tok(log_probs, old_log_probs, advantages, rollout_log_probs, row_aux, params);
    const NormArg na = norm_arg(&params->norm);
    if (!gspo && !use_is)
      launch_partial_grad(mask_dtype, rows, mask, PlainPolicyTok{tok}, partial, n_chunks, g_store, na, 1.0f, s);
    else
      launch_partial_grad(mask_dtype, rows, mask, tok, partial, n_chunks, g_store, na, 1.0f, s);
    ORLHF_CHECK_LAUNCH("orlhf_policy_loss_fwd(partial)");
  }
  const int mode = (params->token_level && !gspo) ? ORLHF_AGG_TOKEN_MEAN : ORLHF_AGG_SEQ_MEAN;
  const int n_out = (use_is && !gspo) ? 4 : 3;
  launch_final<5>(n_rows, n_chunks, partial, mode, norm_arg(&params->norm), 1.0f, n_out, out4, row_coef, s);
  ORLHF_CHECK_LAUNCH("orlhf_policy_loss_fwd(final)");
  return ORLHF_OK;
}

extern "C" int orlhf_policy_loss_fwd(const float* log_probs, const float* old_log_probs, const float* advantages,
                                     const void* mask, int mask_dtype, const float* rollout_log_probs,
                                     int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                                     const orlhf_policy_params* params, void* workspace, float* out4,
                                     float* row_coef, float* row_aux, orlhf_stream_t stream) {
  return policy_loss_fwd_impl(log_probs, old_log_probs, advantages, mask, mask_dtype, rollout_log_probs, n_rows,
                              n_cols, cu_seqlens, params, workspace, out4, row_coef, row_aux, nullptr, stream);
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// Partial sums of orlhf_policy_loss_fwd_noalloc live in this file-scope device array instead of a
// caller-provided workspace. Every GPU the library runs on holds its own copy at its own address,
// taken once per device with hipGetSymbolAddress; host code only ever uses that address.
static __device__ __align__(256) unsigned char scratch[ORLHF_NOALLOC_SCRATCH_BYTES];

namespace orlhf {
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the current device (looked up on the first call per device). The kernels
// run on `stream`'s device: a stream of another device than the current one would be handed the
// current device's address, so that is refused.
static int scratch_on_current_device(hipStream_t stream, void** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(ORLHF_ERR_LAUNCH, "policy_loss_fwd_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices)
    return fail(ORLHF_ERR_UNSUPPORTED, "policy_loss_fwd_noalloc: device index %d outside [0, %d)", device, kMaxDevices);
  if (stream != nullptr) {
    int stream_device = -1;
    e = hipStreamGetDevice(stream, &stream_device);
    if (e != hipSuccess)
      return fail(ORLHF_ERR_LAUNCH, "policy_loss_fwd_noalloc: hipStreamGetDevice: %s", hipGetErrorString(e));
    if (stream_device != device)
      return fail(ORLHF_ERR_INVALID_ARG, "policy_loss_fwd_noalloc: the stream belongs to device %d, the current device is %d",
                  stream_device, device);
  }
  void* p = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(ORLHF_ERR_LAUNCH, "policy_loss_fwd_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", device,
                  hipGetErrorString(e));
    g_scratch_ptr[device].store(p, std::memory_order_release);
  }
  *out = p;
  return ORLHF_OK;
}
}  // namespace orlhf

extern "C" int orlhf_policy_loss_fwd_noalloc(const float* log_probs, const float* old_log_probs,
                                             const float* advantages, const void* mask, int mask_dtype,
                                             const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                                             const int64_t* cu_seqlens, const orlhf_policy_params* params,
                                             float* out4, float* row_coef, float* row_aux,
                                             orlhf_stream_t stream) {
  if (int rc = check_rows("policy_loss_fwd_noalloc", n_rows, n_cols, mask, mask_dtype)) return rc;
  const int64_t need = orlhf_token_workspace_bytes(n_rows, n_cols);
  if (need > (int64_t)ORLHF_NOALLOC_SCRATCH_BYTES)
    return fail(ORLHF_ERR_UNSUPPORTED,
                "policy_loss_fwd_noalloc: %lld rows x %lld columns need %lld bytes of partial sums, the built-in "
                "scratch holds %lld; use orlhf_policy_loss_fwd with a workspace",
                (long long)n_rows, (long long)n_cols, (long long)need, (long long)ORLHF_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = scratch_on_current_device((hipStream_t)stream, &ws)) return rc;
  // every (row, chunk) partial the later stages read is written by the first stage of this call:
  // nothing in the scratch has to start at zero
  return policy_loss_fwd_impl(log_probs, old_log_probs, advantages, mask, mask_dtype, rollout_log_probs, n_rows,
                              n_cols, cu_seqlens, params, ws, out4, row_coef, row_aux, nullptr, stream);
}

extern "C" int orlhf_policy_loss_fwd_grad(const float* log_probs, const float* old_log_probs,
                                          const float* advantages, const void* mask, int mask_dtype,
                                          const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                                          const int64_t* cu_seqlens, const orlhf_policy_params* params,
                                          void* workspace, float* out4, float* row_coef, float* row_aux,
                                          float* g_log_probs, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(params != nullptr && g_log_probs != nullptr, "policy_loss_fwd_grad: NULL params / g_log_probs");
  ORLHF_CHECK_ARG(params->token_level && params->policy_type == ORLHF_POLICY_PPO && norm_given(&params->norm),
                  "policy_loss_fwd_grad: needs the token mean over a given count (token_level, PPO, norm value or "
                  "device scalar); other modes learn a token's weight only after the pass");
  return policy_loss_fwd_impl(log_probs, old_log_probs, advantages, mask, mask_dtype, rollout_log_probs, n_rows,
                              n_cols, cu_seqlens, params, workspace, out4, row_coef, row_aux, g_log_probs, stream);
}

extern "C" int orlhf_policy_loss_bwd(const float* g_out, const float* log_probs, const float* old_log_probs,
                                     const float* advantages, const void* mask, int mask_dtype,
                                     const float* rollout_log_probs, int64_t n_rows, int64_t n_cols,
                                     const int64_t* cu_seqlens, const orlhf_policy_params* params,
                                     const float* row_coef, const float* row_aux, void* workspace,
                                     float* g_log_probs, orlhf_stream_t stream) {
  if (int rc = check_rows("policy_loss_bwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  if (int rc = check_policy("policy_loss_bwd", params, rollout_log_probs)) return rc;
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(g_out && log_probs && old_log_probs && advantages && row_coef && row_aux && g_log_probs,
                  "policy_loss_bwd: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  PolicyTok tok = policy_tok(log_probs, old_log_probs, advantages, rollout_log_probs, row_aux, params);
  if (!tok.gspo) {
    if (tok.is_mode == ORLHF_IS_NONE)
      launch_grad(mask_dtype, rows, mask, PlainPolicyTok{tok}, g_out, 0, row_coef, g_log_probs, s);
    else
      launch_grad(mask_dtype, rows, mask, tok, g_out, 0, row_coef, g_log_probs, s);
    ORLHF_CHECK_LAUNCH("orlhf_policy_loss_bwd");
    return ORLHF_OK;
  }
  ORLHF_CHECK_ARG(workspace != nullptr, "policy_loss_bwd: GSPO needs a workspace");
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  GspoGradTok gt{tok};
  launch_partial(mask_dtype, rows, mask, gt, partial, n_chunks, s);
  ORLHF_CHECK_LAUNCH("orlhf_policy_loss_bwd(gspo partial)");
  const dim3 grid = row_grid(rows), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                       \
  hipLaunchKernelGGL(gspo_grad_kernel<M>, grid, block, 0, s, rows, mask, partial, n_chunks, g_out, row_coef, row_aux, \
                     g_log_probs)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
  ORLHF_CHECK_LAUNCH("orlhf_policy_loss_bwd(gspo grad)");
  return ORLHF_OK;
}

static int value_loss_fwd_impl(const float* values, const float* old_values, const float* returns,
                               const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                               const int64_t* cu_seqlens, int has_clip, float clip_eps, int token_level,
                               const orlhf_norm* norm, void* workspace, float* out2, float* row_coef,
                               float* g_store, orlhf_stream_t stream) {
  if (int rc = check_rows("value_loss_fwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(out2 && workspace, "value_loss_fwd: NULL out / workspace");
  ORLHF_CHECK_ARG((values && returns && (old_values || !has_clip)) || n_rows * n_cols == 0, "value_loss_fwd: NULL input");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  const int n_chunks = (int)chunks_of(rows);
  double* partial = (double*)workspace;
  if (n_rows > 0) {
    ValueTok tok{values, old_values, returns, has_clip, clip_eps};
    launch_partial_grad(mask_dtype, rows, mask, tok, partial, n_chunks, g_store, norm_arg(norm), 0.5f, s);
    ORLHF_CHECK_LAUNCH("orlhf_value_loss_fwd(partial)");
  }
  launch_final<3>(n_rows, n_chunks, partial, token_level ? ORLHF_AGG_TOKEN_MEAN : ORLHF_AGG_SEQ_MEAN, norm_arg(norm),
                  0.5f, 2, out2, row_coef, s);
  ORLHF_CHECK_LAUNCH("orlhf_value_loss_fwd(final)");
  return ORLHF_OK;
}

extern "C" int orlhf_value_loss_fwd(const float* values, const float* old_values, const float* returns,
                                    const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                                    const int64_t* cu_seqlens, int has_clip, float clip_eps, int token_level,
                                    const orlhf_norm* norm, void* workspace, float* out2, float* row_coef,
                                    orlhf_stream_t stream) {
  return value_loss_fwd_impl(values, old_values, returns, mask, mask_dtype, n_rows, n_cols, cu_seqlens, has_clip,
                             clip_eps, token_level, norm, workspace, out2, row_coef, nullptr, stream);
}

extern "C" int orlhf_value_loss_fwd_grad(const float* values, const float* old_values, const float* returns,
                                         const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                                         const int64_t* cu_seqlens, int has_clip, float clip_eps,
                                         const orlhf_norm* norm, void* workspace, float* out2, float* row_coef,
                                         float* g_values, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(g_values != nullptr, "value_loss_fwd_grad: NULL g_values");
  ORLHF_CHECK_ARG(norm_given(norm), "value_loss_fwd_grad: needs the token mean over a given count (norm value or "
                                    "device scalar); other modes learn a token's weight only after the pass");
  return value_loss_fwd_impl(values, old_values, returns, mask, mask_dtype, n_rows, n_cols, cu_seqlens, has_clip,
                             clip_eps, 1, norm, workspace, out2, row_coef, g_values, stream);
}

extern "C" int orlhf_value_loss_bwd(const float* g_out, const float* values, const float* old_values,
                                    const float* returns, const void* mask, int mask_dtype, int64_t n_rows,
                                    int64_t n_cols, const int64_t* cu_seqlens, int has_clip, float clip_eps,
                                    const float* row_coef, float* g_values, orlhf_stream_t stream) {
  if (int rc = check_rows("value_loss_bwd", n_rows, n_cols, mask, mask_dtype)) return rc;
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(g_out && values && returns && (old_values || !has_clip) && row_coef && g_values,
                  "value_loss_bwd: NULL pointer");
  const Rows rows = make_rows(n_rows, n_cols, cu_seqlens);
  ValueTok tok{values, old_values, returns, has_clip, clip_eps};
  launch_grad(mask_dtype, rows, mask, tok, g_out, 0, row_coef, g_values, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_value_loss_bwd");
  return ORLHF_OK;
}
