// Fused lm-head + log-prob / entropy for gfx950: the logits x = hidden @ W^T are produced tile by
// tile on the matrix cores and consumed on the spot, so the [N, V] logits never exist in memory.
//
// Forward: a workgroup owns one 256 x 256 tile of the logits
// (vocabulary x tokens, so that one lane holds 64 vocabulary entries of ONE token per MFMA column):
// it multiplies W[tile] * hidden[block]^T over the hidden dimension and folds the tile into
// per-token statistics (max, sum e^(x-m), sum e^(x-m) x, the same at temperature T, and the
// label's logit), all in registers; 16 bytes per (tile, token) leave the chip. The tiles of a
// token are combined by a small second kernel.
//
// Backward: the vocabulary is cut into chunks of Vc columns. Per chunk, (1) the logits tiles are
// recomputed and turned into P = d(loss)/d(logits) in the 16-bit dtype (the rounding the
// reference's 16-bit logits gradient has), written to a [N, Vc] workspace; (2) dHidden += P @
// W[chunk] and (3) dW[chunk] = P^T @ hidden run on the same matrix-core tile, which reads operands
// in either orientation, so no matrix is ever transposed in memory. Only the chunk of P exists at
// any time (it is written once and read twice, mostly from the Infinity Cache).
#include "mfma_gemm.h"
#include "vocab_rows.h"

namespace orlhf {
namespace lm {

using mm::f32x16;
using mm::Operand;

// "no value yet" / "not a vocabulary entry". Small enough that e^(kLow - m) is 0 for any real m,
// large enough that kLow * log2(e) / T stays finite: a lane whose part of a tile lies wholly past
// the vocabulary keeps (m = kLow, finite sums) and is weighted out exactly when it is merged.
constexpr float kLow = -1.0e30f;
constexpr int kRec = 4;            // floats per (vocabulary tile, token) record: m, s1, t1, sT

// Vocabulary offset of accumulator register r of MFMA row-tile mt inside a wave's 128 rows, minus
// the lane-dependent 4 * (lane >> 5): a compile-time constant per register.
__device__ __forceinline__ constexpr int reg_off(int mt, int r) { return mt * 32 + 8 * (r >> 2) + (r & 3); }

struct Running {
  float m, s1, t1, sT, xl;
};

// Folds one 256 x 256 logits tile into the running statistics of this lane's four tokens.
// vrem = number of valid vocabulary entries from this lane's first row of the tile on (<= 0: none).
template <bool BOTH_T, bool EDGE>
__device__ __forceinline__ void fold_tile(const f32x16 (&acc)[4][4], Running (&run)[4], const int (&lab_rel)[4], int vrem,
                                          float c1, float cT) {
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    float mx = kLow;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float x = (!EDGE || reg_off(mt, r) < vrem) ? acc[mt][nt][r] : kLow;
        mx = fmaxf(mx, x);
      }
    }
    const float m_new = fmaxf(run[nt].m, mx);
    const float n1 = -m_new * c1, nT = -m_new * cT;
    float s1[2] = {0.0f, 0.0f}, t1[2] = {0.0f, 0.0f}, sT[2] = {0.0f, 0.0f};
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        // entries past the vocabulary (EDGE tiles only) contribute exact zeros, also when the lane
        // has seen no real entry yet and m_new is still kLow
        const bool real = !EDGE || reg_off(mt, r) < vrem;
        const float x = real ? acc[mt][nt][r] : 0.0f;
        const float e = real ? fast_exp2(fmaf(x, c1, n1)) : 0.0f;
        s1[r & 1] += e;
        t1[r & 1] = fmaf(e, x, t1[r & 1]);
        if (BOTH_T) sT[r & 1] += real ? fast_exp2(fmaf(x, cT, nT)) : 0.0f;
      }
    }
    // the label's logit: per token one lane of one tile of the vocabulary holds it, so the 64-way
    // selection sits behind a branch that almost every wave skips
    if (lab_rel[nt] >= 0) {
      float xl = run[nt].xl;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) xl = (lab_rel[nt] == reg_off(mt, r)) ? acc[mt][nt][r] : xl;
      }
      run[nt].xl = xl;
    }
    const float d = run[nt].m - m_new;  // <= 0
    const float q1 = fast_exp2(d * c1);
    run[nt].s1 = fmaf(run[nt].s1, q1, s1[0] + s1[1]);
    run[nt].t1 = fmaf(run[nt].t1, q1, t1[0] + t1[1]);
    if (BOTH_T) run[nt].sT = fmaf(run[nt].sT, fast_exp2(d * cT), sT[0] + sT[1]);
    run[nt].m = m_new;
  }
}

__device__ __forceinline__ void merge(Running& a, const Running& b, float c1, float cT, bool both_t) {
  const float m = fmaxf(a.m, b.m);
  const float qa = fast_exp2((a.m - m) * c1), qb = fast_exp2((b.m - m) * c1);
  a.s1 = a.s1 * qa + b.s1 * qb;
  a.t1 = a.t1 * qa + b.t1 * qb;
  if (both_t) a.sT = a.sT * fast_exp2((a.m - m) * cT) + b.sT * fast_exp2((b.m - m) * cT);
  a.xl = fmaxf(a.xl, b.xl);
  a.m = m;
}

// ---------------------------------------------------------------- forward: logits tiles -> statistics
// One workgroup per (vocabulary tile, token block): the tile's statistics of each of its 256 tokens
// go to records[vt][token] = {m, s1, t1, sT}; the lane that holds a token's label writes its logit.
template <int DT, bool BOTH_T>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_fwd_kernel(Operand w, Operand h, const int64_t* __restrict__ labels,
                                                                     float c1, float cT, float* __restrict__ records,
                                                                     float* __restrict__ x_label, int64_t n_token_blocks,
                                                                     int64_t n_vocab_tiles) {
  extern __shared__ __align__(16) char lds[];
  const int64_t n_items = n_token_blocks * n_vocab_tiles;
  const int64_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  int64_t tb, vt;
  mm::grouped_tile(item, n_token_blocks, n_vocab_tiles, tb, vt);
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, wm = wave & 1u, wn = wave >> 1;
  const int64_t n_tokens = h.rows, vocab = w.rows;

  f32x16 acc[4][4];
  mm::tile_product<DT, false, false>(acc, w, h, vt * 256, tb * 256, lds);

  const int64_t vbase = vt * 256 + wm * 128 + 4 * (lane >> 5);  // vocabulary index of this lane's register offset 0
  Running run[4];
  int lab_rel[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    run[nt] = Running{kLow, 0.0f, 0.0f, 0.0f, kLow};
    const int64_t tok = tb * 256 + mm::acc_col(wn, nt, lane);
    const int64_t d = ((labels != nullptr && tok < n_tokens) ? labels[tok] : -1) - vbase;
    lab_rel[nt] = (d >= 0 && d < 128) ? (int)d : -1;
  }
  if (vt * 256 + 256 <= vocab) {
    fold_tile<BOTH_T, false>(acc, run, lab_rel, 128, c1, cT);
  } else {
    const int64_t left = vocab - vbase;
    fold_tile<BOTH_T, true>(acc, run, lab_rel, left > 128 ? 128 : (left < 0 ? 0 : (int)left), c1, cT);
  }
  // the two lane halves and the two waves along the vocabulary hold parts of the same tokens
  __syncthreads();  // every wave is done with the slab buffers: they serve as the exchange area now
  float* ex = (float*)lds;  // [2 wn][4 tokens][32 lanes][4 fields]
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    if (run[nt].xl != kLow) {  // exactly one lane of the grid holds a token's label
      const int64_t tok = tb * 256 + mm::acc_col(wn, nt, lane);
      if (tok < n_tokens) x_label[tok] = run[nt].xl;
    }
    Running o;
    o.m = __shfl_xor(run[nt].m, 32, kWave);
    o.s1 = __shfl_xor(run[nt].s1, 32, kWave);
    o.t1 = __shfl_xor(run[nt].t1, 32, kWave);
    o.sT = __shfl_xor(run[nt].sT, 32, kWave);
    o.xl = kLow;
    merge(run[nt], o, c1, cT, BOTH_T);
    if (wm == 1 && lane < 32) *(f32x4*)(ex + ((wn * 4 + nt) * 32 + lane) * 4) = f32x4{run[nt].m, run[nt].s1, run[nt].t1, run[nt].sT};
  }
  __syncthreads();
  if (wm == 0 && lane < 32) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const f32x4 p = *(const f32x4*)(ex + ((wn * 4 + nt) * 32 + lane) * 4);
      const Running o{p[0], p[1], p[2], p[3], kLow};
      merge(run[nt], o, c1, cT, BOTH_T);
      const int64_t tok = tb * 256 + mm::acc_col(wn, nt, lane);
      if (tok < n_tokens) *(f32x4*)(records + (vt * n_tokens + tok) * kRec) = f32x4{run[nt].m, run[nt].s1, run[nt].t1, run[nt].sT};
    }
  }
}

// ---------------------------------------------------------------- forward: vocabulary ranges -> outputs
constexpr int kCombineBlock = 1024;  // 16 waves: lane = token, the waves split the vocabulary tiles

__global__ __launch_bounds__(kCombineBlock) void lmhead_combine_kernel(const float* __restrict__ records,
                                                                       const float* __restrict__ x_label, int64_t n_tokens,
                                                                       int64_t n_tiles, const int64_t* __restrict__ labels,
                                                                       int64_t vocab, double temperature, int both_t,
                                                                       float* __restrict__ logprob, float* __restrict__ entropy,
                                                                       float* __restrict__ row_stats) {
  constexpr int kWaves = kCombineBlock / kWave;
  __shared__ f32x4 lds[kWaves][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t tok = (int64_t)blockIdx.x * kWave + lane;
  const float c1 = kLog2e, cT = (float)(1.4426950408889634 / temperature);
  Running run{kLow, 0.0f, 0.0f, 0.0f, kLow};
  if (tok < n_tokens) {
    for (int64_t t = wave; t < n_tiles; t += kWaves) {  // 64 consecutive tokens of one tile: one 1 KiB read per wave
      const f32x4 rec = *(const f32x4*)(records + (t * n_tokens + tok) * kRec);
      merge(run, Running{rec[0], rec[1], rec[2], rec[3], kLow}, c1, cT, both_t != 0);
    }
  }
  lds[wave][lane] = f32x4{run.m, run.s1, run.t1, run.sT};
  __syncthreads();
  if (wave != 0 || tok >= n_tokens) return;
  // the 16 partial results of this token, folded in fp64
  float m = kLow;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) m = fmaxf(m, lds[w][lane][0]);
  const double inv_t = 1.0 / temperature;
  double s1 = 0.0, t1 = 0.0, sT = 0.0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const f32x4 rec = lds[w][lane];
    const double d = (double)rec[0] - (double)m;
    const double q1 = exp(d);
    s1 += (double)rec[1] * q1;
    t1 += (double)rec[2] * q1;
    if (both_t) sT += (double)rec[3] * exp(d * inv_t);
  }
  const double lse1 = (double)m + log(s1);
  const double lseT = both_t ? (double)m * inv_t + log(sT) : lse1;
  const double ex = t1 / s1;
  if (logprob != nullptr) {
    const int64_t label = labels[tok];
    float lp;
    if (label >= 0 && label < vocab)
      lp = (float)((double)x_label[tok] * inv_t - lseT);
    else
      lp = (label == -100) ? 0.0f : NAN;
    logprob[tok] = lp;
  }
  if (entropy != nullptr) entropy[tok] = (float)(lse1 - ex);
  if (row_stats != nullptr) *(f32x4*)(row_stats + tok * 4) = f32x4{(float)lseT, (float)lse1, (float)ex, 0.0f};
}

// ---------------------------------------------------------------- backward (1): logits tiles -> P chunk
// P[tok][v - v0] = g_lp * (1[v == label] - softmax(x/T)) / T + g_ent * softmax(x) * (E[x] - x), rounded to DT.
template <int DT, bool BOTH_T>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_bwd_p_kernel(Operand w, Operand h, const int64_t* __restrict__ labels,
                                                                       double temperature,
                                                                       const float* __restrict__ g_logprob,
                                                                       const float* __restrict__ g_entropy,
                                                                       const float* __restrict__ row_stats,
                                                                       uint16_t* __restrict__ p_chunk, int64_t ldp,
                                                                       int64_t v0, int64_t n_token_blocks,
                                                                       int64_t n_chunk_tiles) {
  extern __shared__ __align__(16) char lds[];
  using E = Elt<DT>;
  constexpr int MODE = BOTH_T ? kBwdBothT : kBwdBothT1;
  const int64_t n_items = n_token_blocks * n_chunk_tiles;
  const int64_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  int64_t tb, ct;
  mm::grouped_tile(item, n_token_blocks, n_chunk_tiles, tb, ct);
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, wm = wave & 1u, wn = wave >> 1;
  const int64_t n_tokens = h.rows, vocab = w.rows;

  f32x16 acc[4][4];
  mm::tile_product<DT, false, false>(acc, w, h, v0 + ct * 256, tb * 256, lds);

  const double inv_t = 1.0 / temperature;
  const int64_t vbase = v0 + ct * 256 + wm * 128 + 4 * (lane >> 5);
  const int64_t left = vocab - vbase;
  const int vrem = left > 128 ? 128 : (int)left;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int64_t tok = tb * 256 + mm::acc_col(wn, nt, lane);
    if (tok >= n_tokens) continue;
    const float glp = g_logprob != nullptr ? g_logprob[tok] : 0.0f;
    const float gh = g_entropy != nullptr ? g_entropy[tok] : 0.0f;
    const f32x4 st = *(const f32x4*)(row_stats + tok * 4);
    GradFn<MODE> fn;
    fn.cT = (float)(1.4426950408889634 * inv_t);
    fn.c1 = kLog2e;
    fn.negLT = -(float)((double)st[0] * 1.4426950408889634);
    fn.negL1 = -(float)((double)st[1] * 1.4426950408889634);
    fn.a_lp = -(float)((double)glp * inv_t);
    fn.onehot = (float)((double)glp * inv_t);
    fn.gh = gh;
    fn.k1 = gh * st[2] - (MODE == kBwdBothT1 ? glp : 0.0f);
    const int64_t d = (labels != nullptr ? labels[tok] : -1) - vbase;
    const int lab_rel = (d >= 0 && d < 128) ? (int)d : -1;
    const bool dead = glp == 0.0f && gh == 0.0f;  // masked token: exact zeros, whatever its statistics hold
    uint16_t* out = p_chunk + tok * ldp + (ct * 256 + wm * 128 + 4 * (lane >> 5));
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int off = reg_off(mt, g * 4 + k);
          float y = fn.elem(acc[mt][nt][g * 4 + k]);
          if (lab_rel == off) y += fn.onehot;
          v[k] = (dead || off >= vrem) ? 0.0f : y;
        }
        u32x2 pk;
        if (DT == ORLHF_BF16) {
          pk[0] = pack_bf16(v[0], v[1]);
          pk[1] = pack_bf16(v[2], v[3]);
        } else {
          pk[0] = pack_f16(v[0], v[1]);
          pk[1] = pack_f16(v[2], v[3]);
        }
        *(u32x2*)(out + mt * 32 + g * 8) = pk;
      }
    }
  }
}

// ---------------------------------------------------------------- backward (2), (3): the two products
// C[i][j] (fp32, ldc) = or += sum_k A[i][k] * B[j][k] for the tile at (tm, tn).
template <int DT, bool A_MN, bool B_MN, bool ACCUMULATE>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_gemm_f32_kernel(Operand a, Operand b, float* __restrict__ c,
                                                                          int64_t ldc, int64_t tiles_m, int64_t tiles_n) {
  extern __shared__ __align__(16) char lds[];
  const int64_t n_items = tiles_m * tiles_n;
  const int64_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  int64_t tm, tn;
  mm::grouped_tile(item, tiles_m, tiles_n, tm, tn);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, wm = wave & 1u, wn = wave >> 1;
  f32x16 acc[4][4];
  mm::tile_product<DT, A_MN, B_MN>(acc, a, b, tm * 256, tn * 256, lds);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int64_t j = tn * 256 + mm::acc_col(wn, nt, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t i = tm * 256 + mm::acc_row(wm, mt, r, lane);
        if (i < a.rows && j < b.rows) {
          float* p = c + i * ldc + j;
          *p = ACCUMULATE ? *p + acc[mt][nt][r] : acc[mt][nt][r];
        }
      }
    }
  }
}

// C[i][j] (DT, ldc) = sum_k A[i][k] * B[j][k], rounded once.
template <int DT, bool A_MN, bool B_MN>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_gemm_lowp_kernel(Operand a, Operand b, uint16_t* __restrict__ c,
                                                                           int64_t ldc, int64_t tiles_m, int64_t tiles_n) {
  extern __shared__ __align__(16) char lds[];
  using E = Elt<DT>;
  const int64_t n_items = tiles_m * tiles_n;
  const int64_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  int64_t tm, tn;
  mm::grouped_tile(item, tiles_m, tiles_n, tm, tn);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, wm = wave & 1u, wn = wave >> 1;
  f32x16 acc[4][4];
  mm::tile_product<DT, A_MN, B_MN>(acc, a, b, tm * 256, tn * 256, lds);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int64_t j = tn * 256 + mm::acc_col(wn, nt, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t i = tm * 256 + mm::acc_row(wm, mt, r, lane);
        if (i < a.rows && j < b.rows) E::store1((char*)(c + i * ldc + j), acc[mt][nt][r]);
      }
    }
  }
}

template <int DT>
__global__ __launch_bounds__(kBlock) void lmhead_round_kernel(const float* __restrict__ src, int64_t n_rows, int64_t n_cols,
                                                              uint16_t* __restrict__ dst, int64_t ld_dst) {
  using E = Elt<DT>;
  const int64_t n = n_rows * n_cols;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t r = i / n_cols, c = i - r * n_cols;
    E::store1((char*)(dst + r * ld_dst + c), src[i]);
  }
}

// Measurement: the plain product A * B^T of two K-major operands through the tile core, one tile per
// workgroup in the same order as the kernels above; every thread leaves the sum of its 256
// accumulators (tile_sums[tile * 256 + thread]), so nothing but the product is timed and the
// result can still be checked (a tile's sums add up to the sum of its block of A * B^T).
template <int DT, bool RESIDENT_OPERANDS>
__global__ __launch_bounds__(mm::kThreads, 1) void matrix_tile_probe_kernel(Operand a, Operand b, float* __restrict__ tile_sums,
                                                                            int64_t tiles_m, int64_t tiles_n) {
  extern __shared__ __align__(16) char lds[];
  const int64_t n_items = tiles_m * tiles_n;
  const int64_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  int64_t tm, tn;
  mm::grouped_tile(item, tiles_m, tiles_n, tm, tn);
  f32x16 acc[4][4];
  mm::tile_product<DT, false, false, RESIDENT_OPERANDS>(acc, a, b, tm * 256, tn * 256, lds);
  float sum = 0.0f;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[mt][nt][r];
    }
  }
  tile_sums[(tm * tiles_n + tn) * mm::kThreads + threadIdx.x] = sum;
}

// dst[c][r] = src[r][c] for 16-bit elements, 64 x 64 tiles through LDS: the hidden states as
// [H][N] so that the weight gradient's second operand is K-major (straight into LDS) as well.
__global__ __launch_bounds__(kBlock) void lmhead_transpose_kernel(const uint16_t* __restrict__ src, int64_t n_rows,
                                                                  int64_t n_cols, int64_t ld_src, uint16_t* __restrict__ dst,
                                                                  int64_t ld_dst) {
  __shared__ uint16_t tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int64_t r = r0 + ty + 4 * k, c = c0 + tx;
    tile[ty + 4 * k][tx] = (r < n_rows && c < n_cols) ? src[r * ld_src + c] : (uint16_t)0;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int64_t c = c0 + ty + 4 * k, r = r0 + tx;
    if (c < n_cols && r < n_rows) dst[c * ld_dst + r] = tile[tx][ty + 4 * k];
  }
}

template <int DT>
__global__ __launch_bounds__(kBlock) void lmhead_zero_kernel(uint16_t* __restrict__ dst, int64_t n_rows, int64_t n_cols, int64_t ld) {
  const int64_t n = n_rows * n_cols;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t r = i / n_cols, c = i - r * n_cols;
    dst[r * ld + c] = 0;
  }
}

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline unsigned grid_for_items(int64_t items) { return (unsigned)(((items + 7) / 8) * 8); }

template <typename K>
static hipError_t allow_lds(K kernel, int bytes = mm::kLdsBytes) {
  return hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

static int check_operands(const char* what, const void* hidden, const void* weight, int dtype, int64_t n_rows,
                          int64_t hidden_dim, int64_t vocab, int64_t hidden_stride, int64_t weight_stride) {
  if (dtype != ORLHF_BF16 && dtype != ORLHF_F16)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: the matrix-core path takes bf16 or fp16 operands, got dtype %d", what, dtype);
  if (n_rows < 0 || hidden_dim <= 0 || vocab <= 0)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: n_rows=%lld hidden=%lld vocab=%lld", what, (long long)n_rows,
                (long long)hidden_dim, (long long)vocab);
  if (hidden_stride < hidden_dim || weight_stride < hidden_dim)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: row strides %lld/%lld < hidden %lld", what, (long long)hidden_stride,
                (long long)weight_stride, (long long)hidden_dim);
  if (n_rows > 0 && (hidden == nullptr || weight == nullptr)) return fail(ORLHF_ERR_INVALID_ARG, "%s: NULL hidden / weight", what);
  // buffer loads fetch whole dwords: bases on 4 bytes, even strides and an even hidden size
  if ((((uintptr_t)hidden | (uintptr_t)weight) & 3u) != 0 || ((hidden_stride | weight_stride | hidden_dim) & 1) != 0)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: hidden / weight must be 4-byte aligned with even row strides and an even hidden size",
                what);
  if (hidden_stride >= (1ll << 30) || weight_stride >= (1ll << 30))
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: row strides beyond 2^30 elements", what);
  return ORLHF_OK;
}

// Bytes of the forward's workspace: one record per (vocabulary tile, token), then the label logits.
static int64_t records_bytes(int64_t n_rows, int64_t vocab) {
  const int64_t rows = n_rows > 0 ? n_rows : 1;
  return ((vocab + 255) / 256) * rows * kRec * 4 + round_up(rows * 4, 256);
}
// fp32 accumulator of dHidden.
static int64_t dhidden_bytes(int64_t n_rows, int64_t hidden_dim) { return round_up(n_rows * hidden_dim * 4, 256); }
// the transposed hidden states [hidden_dim][ld]: rows padded off the powers of two (a 16 KiB row
// pitch sends every row to the same L2 channels)
static int64_t transposed_ld(int64_t n_rows) { return round_up(n_rows, 8) + 64; }
static int64_t transposed_bytes(int64_t n_rows, int64_t hidden_dim) { return round_up(hidden_dim * transposed_ld(n_rows) * 2, 256); }

// Row pitch of the P chunk [n_rows][chunk_cols]: off the powers of two for the same reason (with
// a pitch of 64 KiB the backward ran 2-4 % slower; 128 to 4224 bytes of padding measure the same)
static int64_t p_chunk_ld(int64_t chunk_cols) { return chunk_cols + 64; }

template <int DT>
static int launch_fwd(const void* hidden, const void* weight, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                      int64_t hidden_stride, int64_t weight_stride, const int64_t* labels, double temperature,
                      float* logprob, float* entropy, float* row_stats, float* records, hipStream_t s) {
  const Operand w{(const uint16_t*)weight, weight_stride, vocab, hidden_dim};
  const Operand h{(const uint16_t*)hidden, hidden_stride, n_rows, hidden_dim};
  const int64_t n_tb = (n_rows + 255) / 256, n_vt = (vocab + 255) / 256;
  float* x_label = records + n_vt * n_rows * kRec;
  const bool both_t = temperature != 1.0;
  const float c1 = kLog2e, cT = (float)(1.4426950408889634 / temperature);
  const dim3 grid(grid_for_items(n_tb * n_vt)), block(mm::kThreads);
  if (both_t) {
    if (allow_lds(lmhead_fwd_kernel<DT, true>) != hipSuccess) return fail(ORLHF_ERR_LAUNCH, "lmhead_fwd: cannot get %d bytes of LDS", mm::kLdsBytes);
    hipLaunchKernelGGL((lmhead_fwd_kernel<DT, true>), grid, block, mm::kLdsBytes, s, w, h, labels, c1, cT, records, x_label, n_tb, n_vt);
  } else {
    if (allow_lds(lmhead_fwd_kernel<DT, false>) != hipSuccess) return fail(ORLHF_ERR_LAUNCH, "lmhead_fwd: cannot get %d bytes of LDS", mm::kLdsBytes);
    hipLaunchKernelGGL((lmhead_fwd_kernel<DT, false>), grid, block, mm::kLdsBytes, s, w, h, labels, c1, cT, records, x_label, n_tb, n_vt);
  }
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_fwd(tiles)");
  hipLaunchKernelGGL(lmhead_combine_kernel, dim3((unsigned)((n_rows + kWave - 1) / kWave)), dim3(kCombineBlock), 0, s, records,
                     x_label, n_rows, n_vt, labels, vocab, temperature, both_t ? 1 : 0, logprob, entropy, row_stats);
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_fwd(combine)");
  return ORLHF_OK;
}

template <int DT>
static int launch_bwd(const void* hidden, const void* weight, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                      int64_t hidden_stride, int64_t weight_stride, const int64_t* labels, double temperature,
                      const float* g_logprob, const float* g_entropy, const float* row_stats, void* grad_hidden,
                      int64_t grad_hidden_stride, void* grad_weight, int64_t grad_weight_stride, char* workspace,
                      int64_t chunk_cols, hipStream_t s) {
  const Operand w{(const uint16_t*)weight, weight_stride, vocab, hidden_dim};
  const Operand h{(const uint16_t*)hidden, hidden_stride, n_rows, hidden_dim};
  float* dh_acc = (float*)workspace;
  uint16_t* h_t = (uint16_t*)(workspace + dhidden_bytes(n_rows, hidden_dim));
  uint16_t* p_chunk = (uint16_t*)(workspace + dhidden_bytes(n_rows, hidden_dim) + transposed_bytes(n_rows, hidden_dim));
  const int64_t ld_t = transposed_ld(n_rows);
  const int64_t n_tb = (n_rows + 255) / 256, tiles_h = (hidden_dim + 255) / 256;
  const bool both_t = temperature != 1.0;
  const dim3 block(mm::kThreads);
  if (allow_lds(lmhead_bwd_p_kernel<DT, true>) != hipSuccess || allow_lds(lmhead_bwd_p_kernel<DT, false>) != hipSuccess ||
      allow_lds(lmhead_gemm_f32_kernel<DT, false, true, false>) != hipSuccess ||
      allow_lds(lmhead_gemm_f32_kernel<DT, false, true, true>) != hipSuccess ||
      allow_lds(lmhead_gemm_lowp_kernel<DT, true, false>) != hipSuccess)
    return fail(ORLHF_ERR_LAUNCH, "lmhead_bwd: cannot get %d bytes of LDS", mm::kLdsBytes);
  if (grad_weight != nullptr) {
    hipLaunchKernelGGL(lmhead_transpose_kernel, dim3((unsigned)((n_rows + 63) / 64), (unsigned)((hidden_dim + 63) / 64)),
                       dim3(kBlock), 0, s, (const uint16_t*)hidden, n_rows, hidden_dim, hidden_stride, h_t, ld_t);
    ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(transpose)");
  }
  for (int64_t v0 = 0; v0 < vocab; v0 += chunk_cols) {
    const int64_t cols = vocab - v0 < chunk_cols ? vocab - v0 : chunk_cols;  // valid vocabulary entries of this chunk
    const int64_t ctiles = (cols + 255) / 256;
    const int64_t ldp = p_chunk_ld(chunk_cols);
    // (1) P chunk
    {
      const dim3 grid(grid_for_items(n_tb * ctiles));
      if (both_t)
        hipLaunchKernelGGL((lmhead_bwd_p_kernel<DT, true>), grid, block, mm::kLdsBytes, s, w, h, labels, temperature,
                           g_logprob, g_entropy, row_stats, p_chunk, ldp, v0, n_tb, ctiles);
      else
        hipLaunchKernelGGL((lmhead_bwd_p_kernel<DT, false>), grid, block, mm::kLdsBytes, s, w, h, labels, temperature,
                           g_logprob, g_entropy, row_stats, p_chunk, ldp, v0, n_tb, ctiles);
      ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(P)");
    }
    // (2) dHidden[n][h] (+)= sum_v P[n][v] * W[v0 + v][h]
    if (grad_hidden != nullptr) {
      const Operand a{p_chunk, ldp, n_rows, ctiles * 256};  // whole tiles: the pad columns hold zeros
      const Operand b{(const uint16_t*)weight + v0 * weight_stride, weight_stride, hidden_dim, cols};
      const dim3 grid(grid_for_items(n_tb * tiles_h));
      if (v0 == 0)
        hipLaunchKernelGGL((lmhead_gemm_f32_kernel<DT, false, true, false>), grid, block, mm::kLdsBytes, s, a, b, dh_acc,
                           hidden_dim, n_tb, tiles_h);
      else
        hipLaunchKernelGGL((lmhead_gemm_f32_kernel<DT, false, true, true>), grid, block, mm::kLdsBytes, s, a, b, dh_acc,
                           hidden_dim, n_tb, tiles_h);
      ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(dHidden)");
    }
    // (3) dW[v0 + v][h] = sum_n P[n][v] * hidden[n][h]
    if (grad_weight != nullptr) {
      const Operand a{p_chunk, ldp, cols, n_rows};
      const Operand b{h_t, ld_t, hidden_dim, n_rows};
      const dim3 grid(grid_for_items(ctiles * tiles_h));
      hipLaunchKernelGGL((lmhead_gemm_lowp_kernel<DT, true, false>), grid, block, mm::kLdsBytes, s, a, b,
                         (uint16_t*)grad_weight + v0 * grad_weight_stride, grad_weight_stride, ctiles, tiles_h);
      ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(dW)");
    }
  }
  if (grad_hidden != nullptr) {
    hipLaunchKernelGGL(lmhead_round_kernel<DT>, dim3(flat_grid(n_rows * hidden_dim, 16384)), dim3(kBlock), 0, s, dh_acc,
                       n_rows, hidden_dim, (uint16_t*)grad_hidden, grad_hidden_stride);
    ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(round)");
  }
  return ORLHF_OK;
}

}  // namespace lm
}  // namespace orlhf

using namespace orlhf;

extern "C" int64_t orlhf_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab, int backward) {
  if (n_rows < 0 || hidden_dim <= 0 || vocab <= 0) return 0;
  if (!backward) return lm::records_bytes(n_rows, vocab);
  // the fp32 dHidden accumulator, the transposed hidden states, and a chunk of P of about 256 MiB
  // (at least one tile column, at most the vocabulary)
  const int64_t rows = n_rows > 0 ? n_rows : 1;
  int64_t cols = ((256ll << 20) / (2 * rows)) / 256 * 256;
  const int64_t vpad = lm::round_up(vocab, 256);
  cols = cols < 256 ? 256 : (cols > vpad ? vpad : cols);
  return lm::dhidden_bytes(n_rows, hidden_dim) + lm::transposed_bytes(n_rows, hidden_dim) + rows * lm::p_chunk_ld(cols) * 2;
}

extern "C" int orlhf_lmhead_logprob_entropy_fwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                                int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                                int64_t weight_stride, const int64_t* labels, double temperature,
                                                float* logprob, float* entropy, float* row_stats, void* workspace,
                                                int64_t workspace_bytes, orlhf_stream_t stream) {
  if (int rc = lm::check_operands("lmhead_logprob_entropy_fwd", hidden, weight, dtype, n_rows, hidden_dim, vocab,
                                  hidden_stride, weight_stride))
    return rc;
  ORLHF_CHECK_ARG(temperature > 0.0 && temperature == temperature, "lmhead_logprob_entropy_fwd: temperature must be > 0");
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(logprob != nullptr || entropy != nullptr || row_stats != nullptr, "lmhead_logprob_entropy_fwd: nothing to compute");
  ORLHF_CHECK_ARG(logprob == nullptr || labels != nullptr, "lmhead_logprob_entropy_fwd: labels is NULL");
  ORLHF_CHECK_ARG(workspace != nullptr && workspace_bytes >= lm::records_bytes(n_rows, vocab),
                  "lmhead_logprob_entropy_fwd: workspace of %lld bytes needed (orlhf_lmhead_workspace_bytes), got %lld",
                  (long long)lm::records_bytes(n_rows, vocab), (long long)workspace_bytes);
  ORLHF_CHECK_ARG(((uintptr_t)workspace & 15u) == 0, "lmhead_logprob_entropy_fwd: workspace must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == ORLHF_BF16)
    return lm::launch_fwd<ORLHF_BF16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                      temperature, logprob, entropy, row_stats, (float*)workspace, s);
  return lm::launch_fwd<ORLHF_F16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                   temperature, logprob, entropy, row_stats, (float*)workspace, s);
}

extern "C" int orlhf_lmhead_logprob_entropy_bwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                                int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                                int64_t weight_stride, const int64_t* labels, double temperature,
                                                const float* g_logprob, const float* g_entropy, const float* row_stats,
                                                void* grad_hidden, int64_t grad_hidden_stride, void* grad_weight,
                                                int64_t grad_weight_stride, void* workspace, int64_t workspace_bytes,
                                                orlhf_stream_t stream) {
  if (int rc = lm::check_operands("lmhead_logprob_entropy_bwd", hidden, weight, dtype, n_rows, hidden_dim, vocab,
                                  hidden_stride, weight_stride))
    return rc;
  ORLHF_CHECK_ARG(temperature > 0.0 && temperature == temperature, "lmhead_logprob_entropy_bwd: temperature must be > 0");
  ORLHF_CHECK_ARG(grad_hidden != nullptr || grad_weight != nullptr, "lmhead_logprob_entropy_bwd: nothing to compute");
  ORLHF_CHECK_ARG(grad_hidden == nullptr || grad_hidden_stride >= hidden_dim, "lmhead_logprob_entropy_bwd: grad_hidden_stride %lld < hidden %lld",
                  (long long)grad_hidden_stride, (long long)hidden_dim);
  ORLHF_CHECK_ARG(grad_weight == nullptr || grad_weight_stride >= hidden_dim, "lmhead_logprob_entropy_bwd: grad_weight_stride %lld < hidden %lld",
                  (long long)grad_weight_stride, (long long)hidden_dim);
  hipStream_t s = (hipStream_t)stream;
  if (n_rows == 0) {  // no token: dW is all zeros, dHidden is empty
    if (grad_weight != nullptr) {
      hipLaunchKernelGGL(lm::lmhead_zero_kernel<ORLHF_BF16>, dim3(flat_grid(vocab * hidden_dim, 16384)), dim3(kBlock), 0, s,
                         (uint16_t*)grad_weight, vocab, hidden_dim, grad_weight_stride);
      ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(zero)");
    }
    return ORLHF_OK;
  }
  ORLHF_CHECK_ARG(row_stats != nullptr && (g_logprob != nullptr || g_entropy != nullptr),
                  "lmhead_logprob_entropy_bwd: row_stats and at least one upstream gradient are needed");
  ORLHF_CHECK_ARG(g_logprob == nullptr || labels != nullptr, "lmhead_logprob_entropy_bwd: labels is NULL");
  const int64_t fixed = lm::dhidden_bytes(n_rows, hidden_dim) + lm::transposed_bytes(n_rows, hidden_dim);
  // the P chunk takes what is left: n_rows rows of p_chunk_ld(cols) elements, cols a multiple of 256
  int64_t cols = workspace != nullptr && workspace_bytes > fixed
                     ? ((workspace_bytes - fixed) / (2 * n_rows) - (lm::p_chunk_ld(0))) / 256 * 256
                     : 0;
  const int64_t vpad = lm::round_up(vocab, 256);
  if (cols > vpad) cols = vpad;
  ORLHF_CHECK_ARG(cols >= 256, "lmhead_logprob_entropy_bwd: workspace of %lld bytes is too small (orlhf_lmhead_workspace_bytes gives %lld)",
                  (long long)workspace_bytes, (long long)orlhf_lmhead_workspace_bytes(n_rows, hidden_dim, vocab, 1));
  ORLHF_CHECK_ARG(((uintptr_t)workspace & 255u) == 0, "lmhead_logprob_entropy_bwd: workspace must be 256-byte aligned");
  if (dtype == ORLHF_BF16)
    return lm::launch_bwd<ORLHF_BF16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                      temperature, g_logprob, g_entropy, row_stats, grad_hidden, grad_hidden_stride,
                                      grad_weight, grad_weight_stride, (char*)workspace, cols, s);
  return lm::launch_bwd<ORLHF_F16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                   temperature, g_logprob, g_entropy, row_stats, grad_hidden, grad_hidden_stride,
                                   grad_weight, grad_weight_stride, (char*)workspace, cols, s);
}

extern "C" int orlhf_matrix_tile_probe(const void* a, const void* b, int dtype, int64_t m, int64_t n, int64_t k,
                                       int64_t lda, int64_t ldb, int resident_operands, float* tile_sums,
                                       orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(dtype == ORLHF_BF16 || dtype == ORLHF_F16, "matrix_tile_probe: dtype %d (bf16 or fp16)", dtype);
  // a leading dimension of 0 makes every row of that operand the same row: all its loads hit the L1
  ORLHF_CHECK_ARG(m > 0 && n > 0 && k > 0 && (lda >= k || lda == 0) && (ldb >= k || ldb == 0),
                  "matrix_tile_probe: m=%lld n=%lld k=%lld lda=%lld ldb=%lld",
                  (long long)m, (long long)n, (long long)k, (long long)lda, (long long)ldb);
  ORLHF_CHECK_ARG(a != nullptr && b != nullptr && tile_sums != nullptr, "matrix_tile_probe: NULL argument");
  ORLHF_CHECK_ARG((((uintptr_t)a | (uintptr_t)b) & 3u) == 0 && ((lda | ldb) & 1) == 0,
                  "matrix_tile_probe: operands need 4-byte aligned bases and even row strides");
  const lm::Operand oa{(const uint16_t*)a, lda, m, k}, ob{(const uint16_t*)b, ldb, n, k};
  const int64_t tiles_m = (m + 255) / 256, tiles_n = (n + 255) / 256;
  const dim3 grid(lm::grid_for_items(tiles_m * tiles_n)), block(mm::kThreads);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_PROBE(DT, RES)                                                                                   \
  {                                                                                                            \
    if (lm::allow_lds(lm::matrix_tile_probe_kernel<DT, RES>) != hipSuccess)                                    \
      return fail(ORLHF_ERR_LAUNCH, "matrix_tile_probe: cannot get %d bytes of LDS", mm::kLdsBytes);           \
    hipLaunchKernelGGL((lm::matrix_tile_probe_kernel<DT, RES>), grid, block, mm::kLdsBytes, s, oa, ob, tile_sums, tiles_m, tiles_n); \
  }
  if (dtype == ORLHF_BF16) {
    if (resident_operands) ORLHF_PROBE(ORLHF_BF16, true) else ORLHF_PROBE(ORLHF_BF16, false)
  } else {
    if (resident_operands) ORLHF_PROBE(ORLHF_F16, true) else ORLHF_PROBE(ORLHF_F16, false)
  }
#undef ORLHF_PROBE
  ORLHF_CHECK_LAUNCH("orlhf_matrix_tile_probe");
  return ORLHF_OK;
}
