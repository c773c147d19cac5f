// Fused lm-head + log-prob / entropy for gfx950: the logits x = hidden @ W^T are produced tile by
// tile on the matrix cores and consumed on the spot, so the [N, V] logits need not exist in memory.
//
// Forward: a workgroup owns one 256 x 256 tile of the logits (vocabulary x tokens, so that one
// lane holds 64 vocabulary entries of ONE token per MFMA column): it multiplies W[tile] *
// hidden[block]^T over the hidden dimension, rounds the tile to the 16-bit dtype (the rounding the
// reference's lm_head output has before its fp32 up-cast) and folds it into per-token statistics
// (max, sum e^(x-m), sum e^(x-m) x, the same at temperature T, and the label's logit), all in
// registers; 16 bytes per (tile, token) leave the chip. The tiles of a token are combined by a
// small second kernel. A caller with memory to spare has the first `kept_cols` vocabulary columns
// of the rounded logits stored as well (they are produced anyway).
//
// Backward: with P = d(loss)/d(logits) in the 16-bit dtype (the dtype the reference's logits
// gradient has), dHidden = P @ W and dW = P^T @ hidden run on the same matrix-core tile, which reads
// operands in either orientation, so no matrix is ever transposed in memory. Over the kept columns
// P is written over the stored logits by a streaming kernel; the rest of the vocabulary is cut into
// chunks whose logits tiles are recomputed (and rounded as in the forward) into a [N, Vc] workspace,
// one chunk at a time. dHidden is continued from chunk to chunk inside the accumulators, so its
// bits do not depend on how the vocabulary was cut.
#include "mfma_gemm.h"
#include "vocab_rows.h"

namespace orlhf {
namespace lm {

using mm::f32x16;
using mm::Operand;

// "no value yet" / "not a vocabulary entry". Small enough that e^(kLow - m) is 0 for any real m,
// large enough that kLow * log2(e) / T stays finite: a lane whose part of a tile lies wholly past
// the vocabulary keeps (m = kLow, finite sums) and is weighted out exactly when it is merged. A
// power of two, so that kLow * c is exact for any c and such a lane's exponents x * c - m * c come
// out as exactly 0 (with a rounded product they would be the rounding error, of the order 1e22).
constexpr float kLow = -0x1p100f;
constexpr int kRec = 4;            // floats per (vocabulary tile, token) record: m, s1, t1, sT

// Vocabulary offset of accumulator register r of MFMA row-tile mt inside a wave's 128 rows, minus
// the lane-dependent 4 * (lane >> 5): a compile-time constant per register.
__device__ __forceinline__ constexpr int reg_off(int mt, int r) { return mt * 32 + 8 * (r >> 2) + (r & 3); }

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  return DT == ORLHF_BF16 ? pack_bf16(a, b) : pack_f16(a, b);
}
template <int DT>
__device__ __forceinline__ float unpack_half(uint32_t w, int hi) {
  if (DT == ORLHF_BF16) return hi ? bf16_hi(w) : bf16_lo(w);
  const f16x2 h = __builtin_bit_cast(f16x2, w);
  return hi ? (float)h[1] : (float)h[0];
}

// One nt column of a wave's quadrant (4 row-tiles x 16 registers = 64 vocabulary entries of one
// token per lane) rounded to the 16-bit dtype: pk[mt][j] = registers (2 j, 2 j + 1) of row-tile mt.
template <int DT>
__device__ __forceinline__ void round_column(const f32x16 (&acc)[4][4], int nt, uint32_t (&pk)[4][8]) {
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int j = 0; j < 8; ++j) pk[mt][j] = pack2<DT>(acc[mt][nt][2 * j], acc[mt][nt][2 * j + 1]);
  }
}

struct Running {
  float m, s1, t1, sT, xl;
};

// Filler of accumulators past the vocabulary in the last vocabulary tile (their weight rows read
// as zeros, so the product leaves what they start with): kLow for bf16, the most negative finite
// number for fp16. e^(filler - m) is exactly 0 for any real m and filler * 0 is 0: such an entry
// contributes nothing, also when the lane has seen no real entry and its maximum is the filler.
template <int DT>
__device__ __forceinline__ constexpr float filler() { return DT == ORLHF_BF16 ? kLow : -65504.0f; }

// Folds one rounded column into the running statistics of its token. One code path for every tile:
// registers past the vocabulary hold the filler.
template <int DT, bool BOTH_T>
__device__ __forceinline__ void fold_column(const uint32_t (&pk)[4][8], Running& run, int lab_rel, float c1, float cT) {
  float x[4][16];
  float mx = kLow;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      x[mt][r] = unpack_half<DT>(pk[mt][r >> 1], r & 1);
      mx = fmaxf(mx, x[mt][r]);
    }
  }
  const float m_new = fmaxf(run.m, mx);
  const float n1 = -m_new * c1, nT = -m_new * cT;
  float s1[2] = {0.0f, 0.0f}, t1[2] = {0.0f, 0.0f}, sT[2] = {0.0f, 0.0f};
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float e = fast_exp2(fmaf(x[mt][r], c1, n1));
      s1[r & 1] += e;
      t1[r & 1] = fmaf(e, x[mt][r], t1[r & 1]);
      if (BOTH_T) sT[r & 1] += fast_exp2(fmaf(x[mt][r], cT, nT));
    }
  }
  // the label's logit: per token one lane of one tile of the vocabulary holds it, so the 64-way
  // selection sits behind a branch that almost every wave skips
  if (lab_rel >= 0) {
    float xl = run.xl;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) xl = (lab_rel == reg_off(mt, r)) ? x[mt][r] : xl;
    }
    run.xl = xl;
  }
  const float d = run.m - m_new;  // <= 0
  const float q1 = fast_exp2(d * c1);
  run.s1 = fmaf(run.s1, q1, s1[0] + s1[1]);
  run.t1 = fmaf(run.t1, q1, t1[0] + t1[1]);
  if (BOTH_T) run.sT = fmaf(run.sT, fast_exp2(d * cT), sT[0] + sT[1]);
  run.m = m_new;
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

// ---------------------------------------------------------------- a tile of 16-bit results leaves in whole rows
// A lane of the tile holds single columns of 32 rows (or, formed transposed, 8-byte pieces of 32
// rows): stored from the registers, every store instruction touches 32-64 rows, and a CU issues a
// few hundred of them per tile at one per 16 cycles. The tile goes through LDS instead (the slab
// buffers are free once the product is done): each lane deposits its 8-byte pieces, and after a
// barrier every 32 lanes pick up one whole 512-byte row of the tile and store it with 16 bytes per
// lane. Rows lie kOutPitch bytes apart: 512 + 8, so that the 32 rows a wave's deposit touches fall
// on 32 different pairs of LDS banks.
constexpr int kOutPitch = 520;
constexpr int kOutBytes = 256 * kOutPitch;  // 133 120: more than the slab buffers (131 072)
constexpr int kExchangeBytes = 8192;        // the forward's per-token statistics of the four waves, behind the tile
constexpr int kLaunchLds = kOutBytes + kExchangeBytes;
static_assert(kOutBytes >= mm::kLdsBytes && kLaunchLds <= 160 * 1024, "dynamic LDS of every matrix-core launch");

// Four consecutive 16-bit results (lo = the first two) of tile row `row` at tile column `col` (a multiple of 4).
__device__ __forceinline__ void deposit4(char* lds, uint32_t row, uint32_t col, uint32_t lo, uint32_t hi) {
  *(u32x2*)(lds + row * kOutPitch + col * 2) = u32x2{lo, hi};
}

// After a barrier: the deposited tile to out[r * ld + c] for r < rows_valid, c < cols_valid (out points
// at the tile's first element). Whole 16-byte pieces where out and ld allow 16-byte stores.
__device__ __forceinline__ void flush_rows(const char* lds, uint16_t* __restrict__ out, int64_t ld, int64_t rows_valid,
                                           int64_t cols_valid) {
  const uint32_t tid = threadIdx.x, piece = tid & 31u, sub = tid >> 5;  // 32 pieces of 8 columns per row, 8 rows per step
  const bool vec = (((uintptr_t)out & 15u) == 0) && ((ld & 7) == 0);
  const int64_t c0 = (int64_t)piece * 8;
#pragma unroll 4
  for (uint32_t step = 0; step < 32; ++step) {
    const uint32_t row = step * 8 + sub;
    if ((int64_t)row >= rows_valid || c0 >= cols_valid) continue;
    const char* src = lds + row * kOutPitch + piece * 16;
    const u32x2 lo = *(const u32x2*)src, hi = *(const u32x2*)(src + 8);
    uint16_t* dst = out + (int64_t)row * ld + c0;
    if (vec && c0 + 8 <= cols_valid) {
      *(u32x4*)dst = u32x4{lo[0], lo[1], hi[0], hi[1]};
    } else {
      const uint32_t w[4] = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (c0 + e < cols_valid) dst[e] = (uint16_t)(e & 1 ? w[e >> 1] >> 16 : w[e >> 1] & 0xffffu);
    }
  }
}

// ---------------------------------------------------------------- forward: logits tiles -> statistics
// One workgroup per (vocabulary tile, token block): the tile's statistics of each of its 256 tokens
// go to records[vt][token] = {m, s1, t1, sT}; the lane that holds a token's label writes its logit.
// Tiles of the first kept_tiles vocabulary tiles also store their rounded logits, token-major.
template <int DT, bool BOTH_T>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_fwd_kernel(Operand w, Operand h, const int64_t* __restrict__ labels,
                                                                     float c1, float cT, float* __restrict__ records,
                                                                     float* __restrict__ x_label, uint16_t* __restrict__ kept,
                                                                     int64_t kept_ld, uint32_t kept_tiles,
                                                                     uint32_t n_token_blocks, uint32_t n_vocab_tiles) {
  extern __shared__ __align__(16) char lds[];
  const uint32_t n_items = n_token_blocks * n_vocab_tiles;
  const uint32_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  uint32_t tb, vt;
  mm::grouped_tile(item, n_token_blocks, n_vocab_tiles, tb, vt);
  const int64_t n_tokens = h.rows, vocab = w.rows;

  f32x16 acc[4][4];
  {
    uint32_t t0 = threadIdx.x;
    asm volatile("" : "+v"(t0));  // opaque: nothing computed for the start values is kept for the epilogue
    const int64_t left = vocab - ((int64_t)vt * 256 + ((t0 >> 6) & 1u) * 128 + 4 * ((t0 & 63u) >> 5));
    // registers past the vocabulary (last vocabulary tile only) start, and stay, at the filler
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float start = reg_off(mt, r) < left ? 0.0f : filler<DT>();
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[mt][nt][r] = start;
      }
    }
  }
  mm::tile_product<DT, false, false, false>(acc, w, h, (int64_t)vt * 256, (int64_t)tb * 256, lds);

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, wm = wave & 1u, wn = wave >> 1;
  const int64_t vbase = (int64_t)vt * 256 + wm * 128 + 4 * (lane >> 5);  // vocabulary index of this lane's register offset 0
  const bool keep = vt < kept_tiles;
  __syncthreads();  // every wave is done with the slab buffers: they serve as the exchange area now
  float* ex = (float*)(lds + kOutBytes);  // [2 wm][2 wn][4 tokens][32 lanes][4 fields], behind the tile of kept logits
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int64_t tok = (int64_t)tb * 256 + mm::acc_col(wn, nt, lane);
    const int64_t d = ((labels != nullptr && tok < n_tokens) ? labels[tok] : -1) - vbase;
    const int lab_rel = (d >= 0 && d < 128) ? (int)d : -1;
    uint32_t pk[4][8];
    round_column<DT>(acc, nt, pk);
    if (keep) {  // the rounded logits of this token (tile row), 4 consecutive vocabulary entries per piece
      const uint32_t row = mm::acc_col(wn, nt, lane);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) deposit4(lds, row, mm::acc_row(wm, mt, 4 * g, lane), pk[mt][2 * g], pk[mt][2 * g + 1]);
      }
    }
    Running run{kLow, 0.0f, 0.0f, 0.0f, kLow};
    fold_column<DT, BOTH_T>(pk, run, lab_rel, c1, cT);
    if (run.xl != kLow && tok < n_tokens) x_label[tok] = run.xl;  // exactly one lane of the grid holds a token's label
    // the two lane halves and the two waves along the vocabulary hold parts of the same tokens
    Running o;
    o.m = __shfl_xor(run.m, 32, kWave);
    o.s1 = __shfl_xor(run.s1, 32, kWave);
    o.t1 = __shfl_xor(run.t1, 32, kWave);
    o.sT = __shfl_xor(run.sT, 32, kWave);
    o.xl = kLow;
    merge(run, o, c1, cT, BOTH_T);
    if (lane < 32) *(f32x4*)(ex + (((wm * 2 + wn) * 4 + nt) * 32 + lane) * 4) = f32x4{run.m, run.s1, run.t1, run.sT};
  }
  __syncthreads();
  // the kept tile leaves in whole token rows of 256 vocabulary entries (the kept array is whole tiles wide)
  if (keep) flush_rows(lds, kept + (int64_t)tb * 256 * kept_ld + (int64_t)vt * 256, kept_ld, n_tokens - (int64_t)tb * 256, 256);
  if (wm == 0 && lane < 32) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const f32x4 mine = *(const f32x4*)(ex + (((0 * 2 + wn) * 4 + nt) * 32 + lane) * 4);
      const f32x4 p = *(const f32x4*)(ex + (((1 * 2 + wn) * 4 + nt) * 32 + lane) * 4);
      Running run{mine[0], mine[1], mine[2], mine[3], kLow};
      merge(run, Running{p[0], p[1], p[2], p[3], kLow}, c1, cT, BOTH_T);
      const int64_t tok = (int64_t)tb * 256 + mm::acc_col(wn, nt, lane);
      if (tok < n_tokens) *(f32x4*)(records + ((int64_t)vt * n_tokens + tok) * kRec) = f32x4{run.m, run.s1, run.t1, run.sT};
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

// ---------------------------------------------------------------- backward (1): logits -> P
// P[tok][v] = g_lp * (1[v == label] - softmax(x/T)) / T + g_ent * softmax(x) * (E[x] - x), rounded to DT,
// from the rounded logits x. The recompute kernel and the in-place kernel build the same GradFn
// from the same per-token inputs and evaluate the same expression on the same rounded logit, so
// a token's P does not depend on which of the two produced it.
template <int MODE>
__device__ __forceinline__ GradFn<MODE> token_grad_fn(const float* __restrict__ row_stats, const float* __restrict__ g_logprob,
                                                     const float* __restrict__ g_entropy, int64_t tok, double inv_t, bool& dead) {
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
  dead = glp == 0.0f && gh == 0.0f;  // masked token: exact zeros, whatever its statistics hold
  return fn;
}

template <int DT, bool BOTH_T>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_bwd_p_kernel(Operand w, Operand h, const int64_t* __restrict__ labels,
                                                                       double temperature,
                                                                       const float* __restrict__ g_logprob,
                                                                       const float* __restrict__ g_entropy,
                                                                       const float* __restrict__ row_stats,
                                                                       uint16_t* __restrict__ p_chunk, int64_t ldp,
                                                                       int64_t v0, uint32_t n_token_blocks,
                                                                       uint32_t n_chunk_tiles) {
  extern __shared__ __align__(16) char lds[];
  constexpr int MODE = BOTH_T ? kBwdBothT : kBwdBothT1;
  const uint32_t n_items = n_token_blocks * n_chunk_tiles;
  const uint32_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  uint32_t tb, ct;
  mm::grouped_tile(item, n_token_blocks, n_chunk_tiles, tb, ct);
  const int64_t n_tokens = h.rows, vocab = w.rows;

  f32x16 acc[4][4];
  mm::tile_product<DT, false, false>(acc, w, h, v0 + (int64_t)ct * 256, (int64_t)tb * 256, lds);

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, wm = wave & 1u, wn = wave >> 1;
  const double inv_t = 1.0 / temperature;
  const int64_t vbase = v0 + (int64_t)ct * 256 + wm * 128 + 4 * (lane >> 5);
  const int64_t left = vocab - vbase;
  const int vrem = left > 128 ? 128 : (int)left;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int64_t tok = (int64_t)tb * 256 + mm::acc_col(wn, nt, lane);
    if (tok >= n_tokens) continue;
    bool dead;
    const GradFn<MODE> fn = token_grad_fn<MODE>(row_stats, g_logprob, g_entropy, tok, inv_t, dead);
    const int64_t d = (labels != nullptr ? labels[tok] : -1) - vbase;
    const int lab_rel = (d >= 0 && d < 128) ? (int)d : -1;
    uint16_t* out = p_chunk + tok * ldp + ((int64_t)ct * 256 + wm * 128 + 4 * (lane >> 5));
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int off = reg_off(mt, g * 4 + k);
          float y = fn.elem(Elt<DT>::round(acc[mt][nt][g * 4 + k]));
          if (lab_rel == off) y += fn.onehot;
          v[k] = (dead || off >= vrem) ? 0.0f : y;
        }
        *(u32x2*)(out + mt * 32 + g * 8) = u32x2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
      }
    }
  }
}

// The same P from stored logits, written over them: one workgroup per (token, stretch of kInplaceCols
// columns), 8 consecutive columns per lane and step. Columns past the vocabulary (the pad of the
// last tile) and tokens without upstream gradient become zeros.
constexpr int kInplaceCols = 8192;

template <int DT, bool BOTH_T>
__global__ __launch_bounds__(kBlock) void lmhead_p_inplace_kernel(uint16_t* __restrict__ kept, int64_t kept_ld, int64_t kept_cols,
                                                                  int64_t n_tokens, int64_t vocab,
                                                                  const int64_t* __restrict__ labels, double temperature,
                                                                  const float* __restrict__ g_logprob,
                                                                  const float* __restrict__ g_entropy,
                                                                  const float* __restrict__ row_stats) {
  constexpr int MODE = BOTH_T ? kBwdBothT : kBwdBothT1;
  using E = Elt<DT>;
  const int64_t stretches = (kept_cols + kInplaceCols - 1) / kInplaceCols;
  const int64_t n_items = n_tokens * stretches;
  for (int64_t item = blockIdx.x; item < n_items; item += gridDim.x) {
    const int64_t tok = item / stretches, c0 = (item - tok * stretches) * kInplaceCols;
    const int64_t c1 = c0 + kInplaceCols < kept_cols ? c0 + kInplaceCols : kept_cols;
    bool dead;
    const GradFn<MODE> fn = token_grad_fn<MODE>(row_stats, g_logprob, g_entropy, tok, 1.0 / temperature, dead);
    const int64_t label = labels != nullptr ? labels[tok] : -1;
    char* row = (char*)(kept + tok * kept_ld);
    for (int64_t c = c0 + (int64_t)threadIdx.x * 8; c < c1; c += kBlock * 8) {  // kept_cols is a multiple of 8
      float x[8];
      if (!dead && c < vocab) {
        E::unpack(load_vec(row + c * 2), x);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float y = fn.elem(x[j]);
          if (c + j == label) y += fn.onehot;
          x[j] = c + j < vocab ? y : 0.0f;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = 0.0f;
      }
      *(u32x4*)(row + c * 2) = E::pack(x);
    }
  }
}

// ---------------------------------------------------------------- backward (2), (3): the two products
// C[i][j] = sum_k A[i][k] * B[j][k] for the tile at (tm, tn). PRELOAD: the accumulators start from
// the fp32 partial sum in c32 (a product continued from an earlier stretch of k). OUT_F32: the sum
// goes back to c32 (ld32); otherwise it is rounded once to DT and stored to c16 (ld16).
//
// ROWS_OUT (dW: thousands of tiles of a depth of only a few thousand, where the exit of a tile is
// several percent of its time): the tile is formed transposed (B's rows along the accumulators'
// register dimension, A's rows along the lanes: the product is symmetric in its operands), so that
// four consecutive registers of a lane are four consecutive columns j of one row of C, and it
// leaves through LDS in whole rows. dHidden, one tile per CU over the whole vocabulary, stores
// from its registers.
template <int DT, bool A_MN, bool B_MN, bool PRELOAD, bool OUT_F32, bool ROWS_OUT = false>
__global__ __launch_bounds__(mm::kThreads, 1) void lmhead_gemm_kernel(Operand a, Operand b, float* __restrict__ c32, int64_t ld32,
                                                                      uint16_t* __restrict__ c16, int64_t ld16,
                                                                      uint32_t tiles_m, uint32_t tiles_n) {
  static_assert(!ROWS_OUT || (!PRELOAD && !OUT_F32), "the row-wise exit is for a 16-bit result of a product begun here");
  extern __shared__ __align__(16) char lds[];
  using E = Elt<DT>;
  const uint32_t n_items = tiles_m * tiles_n;
  const uint32_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  uint32_t tm, tn;
  mm::grouped_tile(item, tiles_m, tiles_n, tm, tn);
  f32x16 acc[4][4];
  if (PRELOAD) {
    // One MFMA tile (16 registers) after the other, each moved into the accumulation registers as
    // soon as it has arrived. Elements outside the matrix are loaded from its last row / column
    // instead of being predicated (their sums are never stored), and the thread index is opaque so
    // that nothing computed here is kept alive for the epilogue across the whole product.
    uint32_t tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const uint32_t lane = tid & 63u, wave = tid >> 6, wm = wave & 1u, wn = wave >> 1;
    const int64_t i_last = a.rows - 1, j_last = b.rows - 1;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int64_t j0 = (int64_t)tn * 256 + mm::acc_col(wn, nt, lane);
      const float* col = c32 + (j0 < j_last ? j0 : j_last);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t i = (int64_t)tm * 256 + mm::acc_row(wm, mt, r, lane);
          acc[mt][nt][r] = col[(i < i_last ? i : i_last) * ld32];
        }
        asm volatile("" : "+a"(acc[mt][nt]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (ROWS_OUT) {
    // transposed: B's rows along the register dimension, A's rows along the lanes
    mm::tile_product<DT, B_MN, A_MN, true>(acc, b, a, (int64_t)tn * 256, (int64_t)tm * 256, lds);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, w_reg = wave & 1u, w_lane = wave >> 1;
    __syncthreads();  // every wave is done with the slab buffers
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const uint32_t row = mm::acc_col(w_lane, nt, lane);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
          deposit4(lds, row, mm::acc_row(w_reg, mt, 4 * g, lane), pack2<DT>(acc[mt][nt][4 * g], acc[mt][nt][4 * g + 1]),
                   pack2<DT>(acc[mt][nt][4 * g + 2], acc[mt][nt][4 * g + 3]));
      }
    }
    __syncthreads();
    flush_rows(lds, c16 + (int64_t)tm * 256 * ld16 + (int64_t)tn * 256, ld16, a.rows - (int64_t)tm * 256,
               b.rows - (int64_t)tn * 256);
    return;
  }
  mm::tile_product<DT, A_MN, B_MN, !PRELOAD>(acc, a, b, (int64_t)tm * 256, (int64_t)tn * 256, lds);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, wm = wave & 1u, wn = wave >> 1;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int64_t j = (int64_t)tn * 256 + mm::acc_col(wn, nt, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t i = (int64_t)tm * 256 + mm::acc_row(wm, mt, r, lane);
        if (i < a.rows && j < b.rows) {
          if (OUT_F32)
            c32[i * ld32 + j] = acc[mt][nt][r];
          else
            E::store1((char*)(c16 + i * ld16 + j), acc[mt][nt][r]);
        }
      }
    }
  }
}

// Measurement: the plain product A * B^T of two K-major operands through the tile core, one tile per
// workgroup in the same order as the kernels above; every thread leaves the sum of its 256
// accumulators (tile_sums[tile * 256 + thread]), so nothing but the product is timed and the
// result can still be checked (a tile's sums add up to the sum of its block of A * B^T).
template <int DT, bool RESIDENT_OPERANDS>
__global__ __launch_bounds__(mm::kThreads, 1) void matrix_tile_probe_kernel(Operand a, Operand b, float* __restrict__ tile_sums,
                                                                            uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __align__(16) char lds[];
  const uint32_t n_items = tiles_m * tiles_n;
  const uint32_t item = mm::xcd_contiguous(blockIdx.x, n_items);
  if (item >= n_items) return;
  uint32_t tm, tn;
  mm::grouped_tile(item, tiles_m, tiles_n, tm, tn);
  f32x16 acc[4][4];
  mm::tile_product<DT, false, false, true, RESIDENT_OPERANDS>(acc, a, b, (int64_t)tm * 256, (int64_t)tn * 256, lds);
  float sum = 0.0f;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[mt][nt][r];
    }
  }
  tile_sums[((int64_t)tm * tiles_n + tn) * mm::kThreads + threadIdx.x] = sum;
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
static hipError_t allow_lds(K kernel, int bytes = kLaunchLds) {
  return hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

static int check_operand(const char* what, const char* name, const void* p, int64_t ld, int64_t min_ld) {
  if (ld < min_ld) return fail(ORLHF_ERR_INVALID_ARG, "%s: %s row stride %lld < %lld", what, name, (long long)ld, (long long)min_ld);
  // buffer loads fetch whole dwords, and offsets inside a slab (up to 255 rows) are 32-bit
  if (((uintptr_t)p & 3u) != 0 || (ld & 1) != 0)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: %s must be 4-byte aligned with an even row stride", what, name);
  if (ld >= mm::kMaxLd) return fail(ORLHF_ERR_UNSUPPORTED, "%s: %s row stride %lld is beyond 2^23 elements", what, name, (long long)ld);
  return ORLHF_OK;
}

static int check_operands(const char* what, const void* hidden, const void* weight, int dtype, int64_t n_rows,
                          int64_t hidden_dim, int64_t vocab, int64_t hidden_stride, int64_t weight_stride) {
  if (dtype != ORLHF_BF16 && dtype != ORLHF_F16)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: the matrix-core path takes bf16 or fp16 operands, got dtype %d", what, dtype);
  if (n_rows < 0 || hidden_dim <= 0 || vocab <= 0)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: n_rows=%lld hidden=%lld vocab=%lld", what, (long long)n_rows,
                (long long)hidden_dim, (long long)vocab);
  if ((hidden_dim & 1) != 0) return fail(ORLHF_ERR_UNSUPPORTED, "%s: the hidden size must be even", what);
  if (n_rows > 0 && (hidden == nullptr || weight == nullptr)) return fail(ORLHF_ERR_INVALID_ARG, "%s: NULL hidden / weight", what);
  if (int rc = check_operand(what, "hidden", hidden, hidden_stride, hidden_dim)) return rc;
  if (int rc = check_operand(what, "weight", weight, weight_stride, hidden_dim)) return rc;
  // tiles are numbered with 32 bits
  const int64_t tiles = ((n_rows + 255) / 256) * ((vocab + 255) / 256);
  if (tiles >= (1ll << 31) - 8 || ((hidden_dim + 255) / 256) * ((vocab + 255) / 256) >= (1ll << 31) - 8)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: more than 2^31 output tiles", what);
  return ORLHF_OK;
}

static int check_kept(const char* what, const void* kept, int64_t kept_cols, int64_t kept_ld, int64_t vocab) {
  if (kept_cols < 0 || (kept_cols & 255) != 0 || kept_cols > round_up(vocab, 256))
    return fail(ORLHF_ERR_INVALID_ARG, "%s: kept_cols=%lld must be a multiple of 256 between 0 and the padded vocabulary %lld", what,
                (long long)kept_cols, (long long)round_up(vocab, 256));
  if (kept_cols == 0) return ORLHF_OK;
  if (kept == nullptr) return fail(ORLHF_ERR_INVALID_ARG, "%s: kept_logits is NULL", what);
  if (((uintptr_t)kept & 15u) != 0 || (kept_ld & 7) != 0)
    return fail(ORLHF_ERR_UNSUPPORTED, "%s: kept_logits must be 16-byte aligned with a row stride that is a multiple of 8", what);
  return check_operand(what, "kept_logits", kept, kept_ld, kept_cols);
}

// Bytes of the forward's workspace: one record per (vocabulary tile, token), then the label logits.
static int64_t records_bytes(int64_t n_rows, int64_t vocab) {
  const int64_t rows = n_rows > 0 ? n_rows : 1;
  return ((vocab + 255) / 256) * rows * kRec * 4 + round_up(rows * 4, 256);
}
// fp32 accumulator of dHidden between the stretches of the vocabulary.
static int64_t dhidden_bytes(int64_t n_rows, int64_t hidden_dim) { return round_up(n_rows * hidden_dim * 4, 256); }

// Row pitch of the P chunk [n_rows][chunk_cols]: off the powers of two (with a pitch of 64 KiB the
// backward ran 2-4 % slower; 128 to 4224 bytes of padding measure the same)
static int64_t p_chunk_ld(int64_t chunk_cols) { return chunk_cols + 64; }

template <int DT>
static int launch_fwd(const void* hidden, const void* weight, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                      int64_t hidden_stride, int64_t weight_stride, const int64_t* labels, double temperature,
                      float* logprob, float* entropy, float* row_stats, void* kept, int64_t kept_cols, int64_t kept_ld,
                      float* records, hipStream_t s) {
  const Operand w{(const uint16_t*)weight, weight_stride, vocab, hidden_dim};
  const Operand h{(const uint16_t*)hidden, hidden_stride, n_rows, hidden_dim};
  const int64_t n_tb = (n_rows + 255) / 256, n_vt = (vocab + 255) / 256;
  float* x_label = records + n_vt * n_rows * kRec;
  const bool both_t = temperature != 1.0;
  const float c1 = kLog2e, cT = (float)(1.4426950408889634 / temperature);
  const dim3 grid(grid_for_items(n_tb * n_vt)), block(mm::kThreads);
  const uint32_t kept_tiles = (uint32_t)(kept_cols / 256);
  if (both_t) {
    if (allow_lds(lmhead_fwd_kernel<DT, true>) != hipSuccess) return fail(ORLHF_ERR_LAUNCH, "lmhead_fwd: cannot get %d bytes of LDS", lm::kLaunchLds);
    hipLaunchKernelGGL((lmhead_fwd_kernel<DT, true>), grid, block, lm::kLaunchLds, s, w, h, labels, c1, cT, records, x_label,
                       (uint16_t*)kept, kept_ld, kept_tiles, (uint32_t)n_tb, (uint32_t)n_vt);
  } else {
    if (allow_lds(lmhead_fwd_kernel<DT, false>) != hipSuccess) return fail(ORLHF_ERR_LAUNCH, "lmhead_fwd: cannot get %d bytes of LDS", lm::kLaunchLds);
    hipLaunchKernelGGL((lmhead_fwd_kernel<DT, false>), grid, block, lm::kLaunchLds, s, w, h, labels, c1, cT, records, x_label,
                       (uint16_t*)kept, kept_ld, kept_tiles, (uint32_t)n_tb, (uint32_t)n_vt);
  }
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_fwd(tiles)");
  hipLaunchKernelGGL(lmhead_combine_kernel, dim3((unsigned)((n_rows + kWave - 1) / kWave)), dim3(kCombineBlock), 0, s, records,
                     x_label, n_rows, n_vt, labels, vocab, temperature, both_t ? 1 : 0, logprob, entropy, row_stats);
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_fwd(combine)");
  return ORLHF_OK;
}

// dHidden (+)= P[:, stretch] * W[stretch, :]: `first` starts the sum, `last` rounds it into grad_hidden.
template <int DT>
static int launch_dhidden(const Operand& p, const Operand& wt, bool first, bool last, float* dh_acc, int64_t hidden_dim,
                          uint16_t* grad_hidden, int64_t grad_hidden_stride, hipStream_t s) {
  const int64_t n_tb = (p.rows + 255) / 256, tiles_h = (hidden_dim + 255) / 256;
  const dim3 grid(grid_for_items(n_tb * tiles_h)), block(mm::kThreads);
#define ORLHF_DH(PRE, F32)                                                                                                   \
  {                                                                                                                           \
    if (allow_lds(lmhead_gemm_kernel<DT, false, true, PRE, F32>) != hipSuccess)                                              \
      return fail(ORLHF_ERR_LAUNCH, "lmhead_bwd: cannot get %d bytes of LDS", lm::kLaunchLds);                                \
    hipLaunchKernelGGL((lmhead_gemm_kernel<DT, false, true, PRE, F32>), grid, block, lm::kLaunchLds, s, p, wt, dh_acc,        \
                       hidden_dim, grad_hidden, grad_hidden_stride, (uint32_t)n_tb, (uint32_t)tiles_h);                      \
  }
  if (first && last) ORLHF_DH(false, false)
  else if (first) ORLHF_DH(false, true)
  else if (last) ORLHF_DH(true, false)
  else ORLHF_DH(true, true)
#undef ORLHF_DH
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(dHidden)");
  return ORLHF_OK;
}

// dW[stretch, :] = P[:, stretch]^T * hidden: both operands as they lie in memory (MN-major).
template <int DT>
static int launch_dweight(const Operand& pt, const Operand& ht, uint16_t* grad_weight, int64_t grad_weight_stride, hipStream_t s) {
  const int64_t tiles_v = (pt.rows + 255) / 256, tiles_h = (ht.rows + 255) / 256;
  const dim3 grid(grid_for_items(tiles_v * tiles_h)), block(mm::kThreads);
  if (allow_lds(lmhead_gemm_kernel<DT, true, true, false, false, true>) != hipSuccess)
    return fail(ORLHF_ERR_LAUNCH, "lmhead_bwd: cannot get %d bytes of LDS", lm::kLaunchLds);
  hipLaunchKernelGGL((lmhead_gemm_kernel<DT, true, true, false, false, true>), grid, block, lm::kLaunchLds, s, pt, ht, nullptr, 0,
                     grad_weight, grad_weight_stride, (uint32_t)tiles_v, (uint32_t)tiles_h);
  ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(dW)");
  return ORLHF_OK;
}

template <int DT>
static int launch_bwd(const void* hidden, const void* weight, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                      int64_t hidden_stride, int64_t weight_stride, const int64_t* labels, double temperature,
                      const float* g_logprob, const float* g_entropy, const float* row_stats, void* kept, int64_t kept_cols,
                      int64_t kept_ld, void* grad_hidden, int64_t grad_hidden_stride, void* grad_weight,
                      int64_t grad_weight_stride, char* workspace, int64_t chunk_cols, hipStream_t s) {
  const Operand w{(const uint16_t*)weight, weight_stride, vocab, hidden_dim};
  const Operand h{(const uint16_t*)hidden, hidden_stride, n_rows, hidden_dim};
  const Operand ht{(const uint16_t*)hidden, hidden_stride, hidden_dim, n_rows};  // hidden^T, MN-major
  float* dh_acc = (float*)workspace;
  uint16_t* p_chunk = (uint16_t*)(workspace + dhidden_bytes(n_rows, hidden_dim));
  const int64_t n_tb = (n_rows + 255) / 256;
  const bool both_t = temperature != 1.0;
  const int64_t vpad = round_up(vocab, 256);
  bool first = true;
  // stretch [v0, v0 + cols_pad) of the vocabulary, its P in `p` (row pitch ldp, pad columns zero)
  auto products = [&](uint16_t* p, int64_t ldp, int64_t v0, int64_t cols_pad) -> int {
    const int64_t cols = vocab - v0 < cols_pad ? vocab - v0 : cols_pad;  // valid vocabulary entries
    const bool last = v0 + cols_pad >= vpad;
    if (grad_hidden != nullptr) {
      const Operand a{p, ldp, n_rows, cols_pad};
      const Operand b{(const uint16_t*)weight + v0 * weight_stride, weight_stride, hidden_dim, cols};  // W[stretch]^T, MN-major
      if (int rc = launch_dhidden<DT>(a, b, first, last, dh_acc, hidden_dim, (uint16_t*)grad_hidden, grad_hidden_stride, s)) return rc;
    }
    if (grad_weight != nullptr) {
      const Operand a{p, ldp, cols, n_rows};  // P[:, stretch]^T, MN-major
      if (int rc = launch_dweight<DT>(a, ht, (uint16_t*)grad_weight + v0 * grad_weight_stride, grad_weight_stride, s)) return rc;
    }
    first = false;
    return ORLHF_OK;
  };
  if (kept_cols > 0) {
    const int64_t stretches = (kept_cols + kInplaceCols - 1) / kInplaceCols;
    const dim3 grid(slot_grid(n_rows * stretches, 1 << 20)), block(kBlock);
    if (both_t)
      hipLaunchKernelGGL((lmhead_p_inplace_kernel<DT, true>), grid, block, 0, s, (uint16_t*)kept, kept_ld, kept_cols, n_rows, vocab,
                         labels, temperature, g_logprob, g_entropy, row_stats);
    else
      hipLaunchKernelGGL((lmhead_p_inplace_kernel<DT, false>), grid, block, 0, s, (uint16_t*)kept, kept_ld, kept_cols, n_rows, vocab,
                         labels, temperature, g_logprob, g_entropy, row_stats);
    ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(P in place)");
    if (int rc = products((uint16_t*)kept, kept_ld, 0, kept_cols)) return rc;
  }
  if (kept_cols < vpad) {
    if (allow_lds(lmhead_bwd_p_kernel<DT, true>) != hipSuccess || allow_lds(lmhead_bwd_p_kernel<DT, false>) != hipSuccess)
      return fail(ORLHF_ERR_LAUNCH, "lmhead_bwd: cannot get %d bytes of LDS", lm::kLaunchLds);
    const int64_t ldp = p_chunk_ld(chunk_cols);
    for (int64_t v0 = kept_cols; v0 < vpad; v0 += chunk_cols) {
      const int64_t cols_pad = vpad - v0 < chunk_cols ? vpad - v0 : chunk_cols;
      const int64_t ctiles = cols_pad / 256;
      const dim3 grid(grid_for_items(n_tb * ctiles)), block(mm::kThreads);
      if (both_t)
        hipLaunchKernelGGL((lmhead_bwd_p_kernel<DT, true>), grid, block, lm::kLaunchLds, s, w, h, labels, temperature, g_logprob,
                           g_entropy, row_stats, p_chunk, ldp, v0, (uint32_t)n_tb, (uint32_t)ctiles);
      else
        hipLaunchKernelGGL((lmhead_bwd_p_kernel<DT, false>), grid, block, lm::kLaunchLds, s, w, h, labels, temperature, g_logprob,
                           g_entropy, row_stats, p_chunk, ldp, v0, (uint32_t)n_tb, (uint32_t)ctiles);
      ORLHF_CHECK_LAUNCH("orlhf_lmhead_logprob_entropy_bwd(P)");
      if (int rc = products(p_chunk, ldp, v0, cols_pad)) return rc;
    }
  }
  return ORLHF_OK;
}

}  // namespace lm
}  // namespace orlhf

using namespace orlhf;

// Columns of P the backward's workspace holds at a time when nothing else is said: about 256 MiB but
// no fewer than 8192 columns (every chunk re-reads and re-writes the fp32 sum of the hidden-state
// gradient, 8 bytes per token and hidden column: with many tokens narrow chunks would spend more
// time on that than on their products), at most what is not kept.
static int64_t default_chunk_cols(int64_t n_rows, int64_t open_cols) {
  const int64_t rows = n_rows > 0 ? n_rows : 1;
  int64_t cols = ((256ll << 20) / (2 * rows)) / 256 * 256;
  cols = cols < 8192 ? 8192 : cols;
  return cols > open_cols ? open_cols : cols;
}

extern "C" int64_t orlhf_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab, int64_t kept_cols,
                                                int backward) {
  if (n_rows < 0 || hidden_dim <= 0 || vocab <= 0 || kept_cols < 0) return 0;
  if (!backward) return lm::records_bytes(n_rows, vocab);
  const int64_t rows = n_rows > 0 ? n_rows : 1;
  const int64_t open_cols = lm::round_up(vocab, 256) - kept_cols;
  if (open_cols <= 0) return 256;  // everything kept: one product per gradient, nothing to carry between launches
  return lm::dhidden_bytes(n_rows, hidden_dim) + rows * lm::p_chunk_ld(default_chunk_cols(n_rows, open_cols)) * 2;
}

extern "C" int orlhf_lmhead_logprob_entropy_fwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                                int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                                int64_t weight_stride, const int64_t* labels, double temperature,
                                                float* logprob, float* entropy, float* row_stats, void* kept_logits,
                                                int64_t kept_cols, int64_t kept_stride, void* workspace,
                                                int64_t workspace_bytes, orlhf_stream_t stream) {
  if (int rc = lm::check_operands("lmhead_logprob_entropy_fwd", hidden, weight, dtype, n_rows, hidden_dim, vocab,
                                  hidden_stride, weight_stride))
    return rc;
  if (int rc = lm::check_kept("lmhead_logprob_entropy_fwd", kept_logits, kept_cols, kept_stride, vocab)) return rc;
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
                                      temperature, logprob, entropy, row_stats, kept_logits, kept_cols, kept_stride,
                                      (float*)workspace, s);
  return lm::launch_fwd<ORLHF_F16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                   temperature, logprob, entropy, row_stats, kept_logits, kept_cols, kept_stride,
                                   (float*)workspace, s);
}

extern "C" int orlhf_lmhead_logprob_entropy_bwd(const void* hidden, const void* weight, int dtype, int64_t n_rows,
                                                int64_t hidden_dim, int64_t vocab, int64_t hidden_stride,
                                                int64_t weight_stride, const int64_t* labels, double temperature,
                                                const float* g_logprob, const float* g_entropy, const float* row_stats,
                                                void* kept_logits, int64_t kept_cols, int64_t kept_stride,
                                                void* grad_hidden, int64_t grad_hidden_stride, void* grad_weight,
                                                int64_t grad_weight_stride, void* workspace, int64_t workspace_bytes,
                                                orlhf_stream_t stream) {
  if (int rc = lm::check_operands("lmhead_logprob_entropy_bwd", hidden, weight, dtype, n_rows, hidden_dim, vocab,
                                  hidden_stride, weight_stride))
    return rc;
  if (int rc = lm::check_kept("lmhead_logprob_entropy_bwd", kept_logits, kept_cols, kept_stride, vocab)) return rc;
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
  // P rows are addressed by the tile with 32-bit offsets like any operand
  const int64_t open_cols = lm::round_up(vocab, 256) - kept_cols;
  const int64_t fixed = lm::dhidden_bytes(n_rows, hidden_dim);
  int64_t cols = 0;
  if (open_cols > 0) {
    // the P chunk takes what is left: n_rows rows of p_chunk_ld(cols) elements, cols a multiple of 256
    cols = workspace != nullptr && workspace_bytes > fixed
               ? ((workspace_bytes - fixed) / (2 * n_rows) - (lm::p_chunk_ld(0))) / 256 * 256
               : 0;
    if (cols > open_cols) cols = open_cols;
    ORLHF_CHECK_ARG(cols >= 256, "lmhead_logprob_entropy_bwd: workspace of %lld bytes is too small (orlhf_lmhead_workspace_bytes gives %lld)",
                    (long long)workspace_bytes, (long long)orlhf_lmhead_workspace_bytes(n_rows, hidden_dim, vocab, kept_cols, 1));
    if (lm::p_chunk_ld(cols) >= mm::kMaxLd) cols = (mm::kMaxLd - 1 - lm::p_chunk_ld(0)) / 256 * 256;
  }
  ORLHF_CHECK_ARG(((uintptr_t)workspace & 255u) == 0, "lmhead_logprob_entropy_bwd: workspace must be 256-byte aligned");
  if (dtype == ORLHF_BF16)
    return lm::launch_bwd<ORLHF_BF16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                      temperature, g_logprob, g_entropy, row_stats, kept_logits, kept_cols, kept_stride,
                                      grad_hidden, grad_hidden_stride, grad_weight, grad_weight_stride, (char*)workspace, cols, s);
  return lm::launch_bwd<ORLHF_F16>(hidden, weight, n_rows, hidden_dim, vocab, hidden_stride, weight_stride, labels,
                                   temperature, g_logprob, g_entropy, row_stats, kept_logits, kept_cols, kept_stride,
                                   grad_hidden, grad_hidden_stride, grad_weight, grad_weight_stride, (char*)workspace, cols, s);
}

// ---------------------------------------------------------------- diagnostics: the tile on its own
extern "C" int orlhf_matrix_tile_product(const void* a, const void* b, int dtype, int64_t m, int64_t n, int64_t k,
                                         int64_t lda, int64_t ldb, int a_mn_major, int b_mn_major, int accumulate,
                                         float* c, int64_t ldc, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(dtype == ORLHF_BF16 || dtype == ORLHF_F16, "matrix_tile_product: dtype %d (bf16 or fp16)", dtype);
  ORLHF_CHECK_ARG(m > 0 && n > 0 && k > 0 && ldc >= n, "matrix_tile_product: m=%lld n=%lld k=%lld ldc=%lld", (long long)m,
                  (long long)n, (long long)k, (long long)ldc);
  ORLHF_CHECK_ARG(a != nullptr && b != nullptr && c != nullptr, "matrix_tile_product: NULL argument");
  if (int rc = lm::check_operand("matrix_tile_product", "a", a, lda, a_mn_major ? m : k)) return rc;
  if (int rc = lm::check_operand("matrix_tile_product", "b", b, ldb, b_mn_major ? n : k)) return rc;
  const lm::Operand oa{(const uint16_t*)a, lda, m, k}, ob{(const uint16_t*)b, ldb, n, k};
  const int64_t tiles_m = (m + 255) / 256, tiles_n = (n + 255) / 256;
  ORLHF_CHECK_ARG(tiles_m * tiles_n < (1ll << 31) - 8, "matrix_tile_product: more than 2^31 output tiles");
  const dim3 grid(lm::grid_for_items(tiles_m * tiles_n)), block(mm::kThreads);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_TP(DT, AM, BM, PRE)                                                                                             \
  {                                                                                                                           \
    if (lm::allow_lds(lm::lmhead_gemm_kernel<DT, AM, BM, PRE, true>) != hipSuccess)                                           \
      return fail(ORLHF_ERR_LAUNCH, "matrix_tile_product: cannot get %d bytes of LDS", lm::kLaunchLds);                        \
    hipLaunchKernelGGL((lm::lmhead_gemm_kernel<DT, AM, BM, PRE, true>), grid, block, lm::kLaunchLds, s, oa, ob, c, ldc, nullptr, 0, \
                       (uint32_t)tiles_m, (uint32_t)tiles_n);                                                                 \
  }
#define ORLHF_TP_LAYOUT(DT, PRE)                                    \
  {                                                                 \
    if (!a_mn_major && !b_mn_major) ORLHF_TP(DT, false, false, PRE) \
    else if (!a_mn_major) ORLHF_TP(DT, false, true, PRE)            \
    else if (!b_mn_major) ORLHF_TP(DT, true, false, PRE)            \
    else ORLHF_TP(DT, true, true, PRE)                              \
  }
  if (dtype == ORLHF_BF16) {
    if (accumulate) ORLHF_TP_LAYOUT(ORLHF_BF16, true) else ORLHF_TP_LAYOUT(ORLHF_BF16, false)
  } else {
    if (accumulate) ORLHF_TP_LAYOUT(ORLHF_F16, true) else ORLHF_TP_LAYOUT(ORLHF_F16, false)
  }
#undef ORLHF_TP_LAYOUT
#undef ORLHF_TP
  ORLHF_CHECK_LAUNCH("orlhf_matrix_tile_product");
  return ORLHF_OK;
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
  if (lda >= mm::kMaxLd || ldb >= mm::kMaxLd)
    return fail(ORLHF_ERR_UNSUPPORTED, "matrix_tile_probe: row strides beyond 2^23 elements");
  const lm::Operand oa{(const uint16_t*)a, lda, m, k}, ob{(const uint16_t*)b, ldb, n, k};
  const int64_t tiles_m = (m + 255) / 256, tiles_n = (n + 255) / 256;
  ORLHF_CHECK_ARG(tiles_m * tiles_n < (1ll << 31) - 8, "matrix_tile_probe: more than 2^31 output tiles");
  const dim3 grid(lm::grid_for_items(tiles_m * tiles_n)), block(mm::kThreads);
  hipStream_t s = (hipStream_t)stream;
#define ORLHF_PROBE(DT, RES)                                                                                   \
  {                                                                                                            \
    if (lm::allow_lds(lm::matrix_tile_probe_kernel<DT, RES>) != hipSuccess)                                    \
      return fail(ORLHF_ERR_LAUNCH, "matrix_tile_probe: cannot get %d bytes of LDS", lm::kLaunchLds);           \
    hipLaunchKernelGGL((lm::matrix_tile_probe_kernel<DT, RES>), grid, block, lm::kLaunchLds, s, oa, ob, tile_sums, (uint32_t)tiles_m, (uint32_t)tiles_n); \
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
