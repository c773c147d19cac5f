// Advantage kernels for gfx950: terminal-reward placement, GAE / discounted returns as a
// parallel reverse-time scan, group baselines and global masked whitening. Forward only.
//
// The scan: A_t = delta_t + c * A_{t+1} is a linear recurrence with a constant coefficient, so a
// lane that owns ITEMS consecutive tokens reduces them to an affine map C -> b + a*C of the
// carry C entering from later tokens. Maps compose associatively; a wave composes its 64 maps with
// log2(64) cross-lane steps, the 4 waves of the workgroup chain through LDS, and a row longer than
// one tile (kBlock * ITEMS tokens) walks its tiles from the end carrying one number. Carries
// and the in-lane recurrence are fp64, inputs and outputs fp32. A lane loads its consecutive
// tokens straight into registers with one 16-byte load per array (the value after them comes from
// the next lane by a shuffle) and stores its outputs the same way; only the per-wave affine
// carries go through LDS.
#include "common.h"

namespace orlhf {


// ---------------------------------------------------------------- compute_reward
template <int MASK_DT>
__device__ __forceinline__ int64_t mask_as_int(const void* mask, int64_t i) {
  if (MASK_DT == ORLHF_MASK_NONE) return 1;
  if (MASK_DT == ORLHF_MASK_U8) return (int64_t)((const uint8_t*)mask)[i];
  if (MASK_DT == ORLHF_MASK_F32) return (int64_t)((const float*)mask)[i];  // .long() truncates
  return ((const int64_t*)mask)[i];
}

template <int MASK_DT>
__device__ __forceinline__ void mask_as_int4(const void* mask, int64_t i0, int64_t* v) {
  if (MASK_DT == ORLHF_MASK_I64) {
    const i64x2e lo = *(const i64x2e*)((const int64_t*)mask + i0), hi = *(const i64x2e*)((const int64_t*)mask + i0 + 2);
    v[0] = lo[0], v[1] = lo[1], v[2] = hi[0], v[3] = hi[1];
  } else {  // bytes are exact as floats; a float mask truncates like .long()
    float m[4];
    load_mask4<MASK_DT>(mask, i0, m);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = (int64_t)m[k];
  }
}

// Index (from the row's first token) of the last position where (int64)mask is maximal: the
// arg-max over the flipped row that the reference takes. Called by the whole workgroup.
template <int MASK_DT>
__device__ __forceinline__ int64_t last_max_of_mask(const RowWalk& rw, int64_t start,
                                                    const void* __restrict__ mask, int64_t* lds_val,
                                                    int64_t* lds_idx) {
  int64_t best_v = INT64_MIN, best_i = -1;
  auto see = [&](int64_t v, int64_t t) {
    if (v > best_v || (v == best_v && t > best_i)) {
      best_v = v;
      best_i = t;
    }
  };
  if (MASK_DT == ORLHF_MASK_U8) {
    // byte masks: 16 tokens per lane and load between the row's first and last 16-byte boundary
    // (a quarter of the steps of the four-token walk; this pass is latency-bound)
    const uint8_t* bytes = (const uint8_t*)mask + start;
    const int64_t len = rw.len;
    int64_t head = (int64_t)((16 - ((uintptr_t)bytes & 15)) & 15);
    head = head < len ? head : len;
    const int64_t groups = (len - head) / 16;
    int best_byte = -1;  // a lane meets its tokens in rising order: >= keeps the last maximum
    for (int64_t t = threadIdx.x; t < head; t += kBlock)
      if ((int)bytes[t] >= best_byte) best_byte = bytes[t], best_i = t;
#pragma unroll 2
    for (int64_t g = threadIdx.x; g < groups; g += kBlock) {
      const u32x4 w = *(const u32x4*)(bytes + head + g * 16);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int v = (int)((w[k / 4] >> (8 * (k % 4))) & 0xffu);
        if (v >= best_byte) best_byte = v, best_i = head + g * 16 + k;
      }
    }
    for (int64_t t = head + groups * 16 + threadIdx.x; t < len; t += kBlock)
      if ((int)bytes[t] >= best_byte) best_byte = bytes[t], best_i = t;
    best_v = best_byte;  // -1 for a lane that saw nothing: below every byte
  } else {
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          int64_t v[4];
          mask_as_int4<MASK_DT>(mask, i0, v);
#pragma unroll
          for (int k = 0; k < 4; ++k) see(v[k], i0 + k - start);
        },
        [&](int64_t i) { see(mask_as_int<MASK_DT>(mask, i), i - start); });
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const int64_t ov = __shfl_xor(best_v, o, kWave);
    const int64_t oi = __shfl_xor(best_i, o, kWave);
    if (ov > best_v || (ov == best_v && oi > best_i)) {
      best_v = ov;
      best_i = oi;
    }
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    lds_val[threadIdx.x / kWave] = best_v;
    lds_idx[threadIdx.x / kWave] = best_i;
  }
  __syncthreads();
  best_v = lds_val[0];
  best_i = lds_idx[0];
#pragma unroll
  for (int w = 1; w < kWavesPerBlock; ++w) {
    if (lds_val[w] > best_v || (lds_val[w] == best_v && lds_idx[w] > best_i)) {
      best_v = lds_val[w];
      best_i = lds_idx[w];
    }
  }
  __syncthreads();
  return best_i;
}

// The sequence reward as the reference places it: clipped when a range is given (NaN passes).
__device__ __forceinline__ float clipped_reward(float rb, int has_clip, float clip_lo, float clip_hi) {
  if (has_clip) rb = (rb != rb) ? rb : fminf(fmaxf(rb, clip_lo), clip_hi);
  return rb;
}

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void compute_reward_kernel(Rows rows, const float* __restrict__ r,
                                                                float neg_coef, const float* __restrict__ kl,
                                                                const void* __restrict__ mask, int has_clip,
                                                                float clip_lo, float clip_hi,
                                                                float* __restrict__ reward,
                                                                int64_t* __restrict__ eos_index) {
  __shared__ int64_t lds_val[kWavesPerBlock];
  __shared__ int64_t lds_idx[kWavesPerBlock];
  const int slot_b = slot_bits(rows.n_rows);
  for (int64_t slot = blockIdx.x; slot < row_slots(rows.n_rows); slot += gridDim.x) {
    const int64_t b = row_of_slot(slot, slot, slot_b);
    if (b >= rows.n_rows) continue;
    int64_t start, len;
    row_span(rows, b, start, len);
    if (len <= 0) {
      if (threadIdx.x == 0 && eos_index != nullptr) eos_index[b] = -1;
      continue;
    }
    const RowWalk rw = row_walk(rows, b);
    const int64_t best_i = last_max_of_mask<MASK_DT>(rw, start, mask, lds_val, lds_idx);
    const float rb = clipped_reward(r[b], has_clip, clip_lo, clip_hi);
    for_row_tokens(
        rw,
        [&](int64_t i0) {
          const f32x4 k4 = stream_load4(kl + i0);
          f32x4 o;
#pragma unroll
          for (int k = 0; k < 4; ++k) o[k] = ((i0 + k - start == best_i) ? rb : 0.0f) + neg_coef * k4[k];
          __builtin_nontemporal_store(o, (f32x4e*)(reward + i0));
        },
        [&](int64_t i) { reward[i] = ((i - start == best_i) ? rb : 0.0f) + neg_coef * kl[i]; });
    if (threadIdx.x == 0 && eos_index != nullptr) eos_index[b] = best_i;
  }
}

// ---------------------------------------------------------------- reverse scan (GAE, returns)
// Tokens per lane and tile (ITEMS below): 4 for GAE (8 is 75 % slower there: registers), 8 for the
// discounted returns with their single input and output (8 % faster than 4).
constexpr int kGaeItems = 4, kReturnItems = 8;

struct Affine {  // C -> b + a * C
  double a, b;
};
// apply `inner` first (later tokens), then `outer` (earlier tokens)
__device__ __forceinline__ Affine compose(const Affine& outer, const Affine& inner) {
  Affine r;
  r.a = outer.a * inner.a;
  r.b = outer.b + outer.a * inner.b;
  return r;
}

// One tile of a row in registers: this lane's ITEMS consecutive tokens, masked, plus the
// value that follows them (the next lane's first; the next tile's first for the last lane).
template <int ITEMS>
struct ScanTile {
  float r[ITEMS];
  float v[ITEMS + 1];
};

// Per-token rewards made on the fly from the KL estimate (REWARD mode of the scan): the token
// reward is neg_coef * kl plus the sequence reward at position `eos` of the walk, as
// compute_reward_kernel writes it; `sum` collects the row's token rewards.
struct RowReward {
  float seq, neg_coef;
  int64_t eos;  // index in the row
  double sum;
};

// The fp32 arrays of one row as buffer resources that end where the row ends: a 16-byte access
// that reaches past the row reads zeros there and stores nothing there (the range check is per
// dword), so the lane that meets the row's end, and the lanes past it, run the same two or three
// instructions as every other lane instead of an element-by-element branch.
struct ScanRow {
  __amdgpu_buffer_rsrc_t rewards, values, adv, ret;
};
template <bool GAE>
__device__ __forceinline__ ScanRow scan_row(const RowWalk& rw, const float* values, const float* rewards, float* adv,
                                            float* ret) {
  // rows hold fewer than 2^30 tokens (host check on the row bound; a longer packed row is cut there)
  const int bytes = (int)(uint32_t)((rw.len < (1ll << 30) - 1 ? rw.len : (1ll << 30) - 1) * 4);
  ScanRow r;
  r.rewards = __builtin_amdgcn_make_buffer_rsrc((void*)(rewards + rw.base), 0, bytes, 0x00020000);
  r.ret = __builtin_amdgcn_make_buffer_rsrc((void*)(ret + rw.base), 0, bytes, 0x00020000);
  r.values = __builtin_amdgcn_make_buffer_rsrc((void*)(GAE ? values + rw.base : rewards + rw.base), 0, bytes, 0x00020000);
  r.adv = __builtin_amdgcn_make_buffer_rsrc((void*)(GAE ? adv + rw.base : ret + rw.base), 0, bytes, 0x00020000);
  return r;
}
constexpr int kNonTemporal = 2;  // cache-policy bits of a buffer access: nt

// Must be called by all lanes of the workgroup (it exchanges the following value across lanes).
// n_total: tokens in the whole arrays (a mask load may read past the row, never past the array).
template <int MASK_DT, bool GAE, bool REWARD, int ITEMS>
__device__ __forceinline__ ScanTile<ITEMS> load_scan_tile(const RowWalk& rw, const ScanRow& row, int64_t tile0, int64_t n_total,
                                                   const float* __restrict__ values,
                                                   const void* __restrict__ mask, RowReward& rr) {
  static_assert(ITEMS == 4 || ITEMS == 8, "a lane's tokens are one or two 16-byte loads");
  ScanTile<ITEMS> t;
  const int64_t p0 = tile0 + (int64_t)threadIdx.x * ITEMS;
  const uint32_t off = (uint32_t)p0 * 4u;
  auto reward_of = [&](float raw, int64_t p) {
    if (!REWARD) return raw;
    const float tok = ((p == rr.eos) ? rr.seq : 0.0f) + rr.neg_coef * raw;
    rr.sum += (double)tok;
    return tok;
  };
#pragma unroll
  for (int q = 0; q < ITEMS / 4; ++q) {
    // two groups per lane share their cache lines: cached loads then (non-temporal ones fetched
    // 47 % more than the rewards and the mask hold)
    const f32x4 r4 = __builtin_bit_cast(
        f32x4, __builtin_amdgcn_raw_buffer_load_b128(row.rewards, off + q * 16u, 0, ITEMS == 4 ? kNonTemporal : 0));
    f32x4 v4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (GAE) v4 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(row.values, off + q * 16u, 0, 0));  // plain: the last lane re-reads across the wave's end
    float m[4];
    if (rw.base + p0 + q * 4 + 4 <= n_total) {  // past the row's end the mask of the next row is read; its tokens are zeros here
      load_mask4<MASK_DT, ITEMS == 4>(mask, rw.base + p0 + q * 4, m);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) m[j] = (p0 + q * 4 + j < rw.len) ? load_mask<MASK_DT>(mask, rw.base + p0 + q * 4 + j) : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool in_row = p0 + q * 4 + j < rw.len;
      t.r[q * 4 + j] = in_row ? m[j] * reward_of(r4[j], p0 + q * 4 + j) : 0.0f;
      t.v[q * 4 + j] = in_row ? m[j] * v4[j] : 0.0f;
    }
  }
  t.v[ITEMS] = 0.0f;
  if (GAE) {
    const float from_next_lane = __shfl_down(t.v[0], 1, kWave);
    const int64_t p = p0 + ITEMS;  // first token of the next wave (or tile) for the last lane
    float after = 0.0f;
    if ((threadIdx.x & (kWave - 1)) == kWave - 1 && p < rw.len)
      after = load_mask<MASK_DT>(mask, rw.base + p) * values[rw.base + p];
    t.v[ITEMS] = (threadIdx.x & (kWave - 1)) == kWave - 1 ? after : from_next_lane;
  }
  return t;
}

// Four consecutive outputs of a lane. GAE's two outputs leave with non-temporal stores (10 %
// faster there; the single output of the returns is faster with plain stores).
template <bool GAE>
__device__ __forceinline__ void store_scan4(const ScanRow& row, uint32_t off, const float* a, const float* r) {
  const f32x4 a4 = {a[0], a[1], a[2], a[3]};
  if (GAE) {
    const f32x4 r4 = {r[0], r[1], r[2], r[3]};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, a4), row.adv, off, 0, kNonTemporal);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, r4), row.ret, off, 0, kNonTemporal);
  } else {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, a4), row.ret, off, 0, 0);
  }
}

// One workgroup per row, walking it backwards in tiles of kScanTile tokens; the tile before the
// current one is loaded (straight into registers, no staging) while the current one is scanned.
// REWARD: `rewards` holds the per-token KL estimate and the token rewards are made from it and
// the sequence rewards `seq` on the fly (compute_reward fused in); reward_sum[b] receives the sum
// of row b's token rewards.
struct SeqReward {
  const float* seq;  // [n_rows]
  float neg_coef;
  int has_clip;
  float clip_lo, clip_hi;
  float* reward_sum;  // [n_rows], nullable
};

template <int MASK_DT, bool GAE, bool REWARD>
__global__ __launch_bounds__(kBlock) void reverse_scan_kernel(Rows rows, const float* __restrict__ values,
                                                              const float* __restrict__ rewards,
                                                              const void* __restrict__ mask, double gamma,
                                                              double coef, SeqReward sr, float* __restrict__ adv,
                                                              float* __restrict__ ret) {
  constexpr int ITEMS = GAE ? kGaeItems : kReturnItems, kScanTile = kBlock * ITEMS;
  __shared__ Affine lds_wave[2][kWavesPerBlock];  // alternating: one barrier per tile is enough
  __shared__ int64_t lds_val[kWavesPerBlock];
  __shared__ int64_t lds_idx[kWavesPerBlock];
  __shared__ double lds_sum[kWavesPerBlock];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;

  double pw[ITEMS + 1];  // coef^k
  pw[0] = 1.0;
#pragma unroll
  for (int k = 1; k <= ITEMS; ++k) pw[k] = pw[k - 1] * coef;

  const int slot_b = slot_bits(rows.n_rows);
  const int64_t n_total = rows.cu != nullptr ? rows.cu[rows.n_rows] : rows.n_rows * rows.n_cols;
  int buf = 0;
  // A caller that knows the row lengths hands the rows out longest first (rows.order): the last
  // workgroups to start then hold the shortest rows, instead of a long row's sequential walk
  // ending alone. Otherwise rows are spread by row_of_slot().
  const int64_t n_slots = rows.order != nullptr ? rows.n_rows : row_slots(rows.n_rows);
  for (int64_t slot = blockIdx.x; slot < n_slots; slot += gridDim.x) {
    const int64_t b = rows.order != nullptr ? rows.order[slot] : row_of_slot(slot, slot, slot_b);
    if (b < 0 || b >= rows.n_rows) continue;
    const RowWalk rw = row_walk(rows, b);
    if (rw.len <= 0) {
      if (REWARD && threadIdx.x == 0 && sr.reward_sum != nullptr) sr.reward_sum[b] = 0.0f;
      continue;
    }
    RowReward rr{0.0f, 0.0f, -1, 0.0};
    if (REWARD) {
      rr.seq = clipped_reward(sr.seq[b], sr.has_clip, sr.clip_lo, sr.clip_hi);
      rr.neg_coef = sr.neg_coef;
      rr.eos = MASK_DT == ORLHF_MASK_NONE  // without a mask the last column is the last maximum
                   ? rw.len - 1
                   : last_max_of_mask<MASK_DT>(rw, rw.base, mask, lds_val, lds_idx);
    }
    const int64_t n_tiles = (rw.len + kScanTile - 1) / kScanTile;
    double tile_carry = 0.0;  // A at the first token of the previous (later) tile
    const ScanRow row = scan_row<GAE>(rw, values, rewards, adv, ret);
    ScanTile<ITEMS> cur =
        load_scan_tile<MASK_DT, GAE, REWARD, ITEMS>(rw, row, (n_tiles - 1) * kScanTile, n_total, values, mask, rr);
    for (int64_t tile = n_tiles - 1; tile >= 0; --tile) {
      const int64_t tile0 = tile * kScanTile;
      ScanTile<ITEMS> nxt = cur;
      if (tile > 0)
        nxt = load_scan_tile<MASK_DT, GAE, REWARD, ITEMS>(rw, row, tile0 - kScanTile, n_total, values, mask, rr);
      // in-lane recurrence with zero carry-in
      double local[ITEMS];
      double run = 0.0;
#pragma unroll
      for (int j = ITEMS - 1; j >= 0; --j) {
        const double delta =
            GAE ? ((double)cur.r[j] + gamma * (double)cur.v[j + 1]) - (double)cur.v[j] : (double)cur.r[j];
        run = delta + coef * run;
        local[j] = run;
      }
      // inclusive suffix composition over the wave: lane i ends with the map of lanes i..63
      Affine f;
      f.a = pw[ITEMS];
      f.b = local[0];
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        Affine o;
        o.a = __shfl_down(f.a, d, kWave);
        o.b = __shfl_down(f.b, d, kWave);
        if (lane + d < kWave) f = compose(f, o);
      }
      if (lane == 0) lds_wave[buf][wave] = f;
      __syncthreads();
      // carry entering this wave = maps of the later waves applied to the tile carry; applying
      // the earlier waves' maps as well gives A at the tile's first token, the next tile's carry
      double wave_carry = tile_carry, c = tile_carry;
#pragma unroll
      for (int w = kWavesPerBlock - 1; w >= 0; --w) {
        c = lds_wave[buf][w].b + lds_wave[buf][w].a * c;
        if (w == wave + 1) wave_carry = c;
      }
      tile_carry = c;
      buf ^= 1;
      // carry entering this lane = A at the first token of lane+1
      Affine after;
      after.a = __shfl_down(f.a, 1, kWave);
      after.b = __shfl_down(f.b, 1, kWave);
      const double carry = (lane == kWave - 1) ? wave_carry : after.b + after.a * wave_carry;
      const int64_t p0 = tile0 + (int64_t)threadIdx.x * ITEMS;
      float out_a[ITEMS], out_r[ITEMS];
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) {
        const double a_t = local[j] + pw[ITEMS - j] * carry;
        out_a[j] = (float)a_t;
        out_r[j] = (float)(a_t + (double)cur.v[j]);
      }
      store_scan4<GAE>(row, (uint32_t)p0 * 4u, out_a, out_r);
      if (ITEMS == 8) store_scan4<GAE>(row, (uint32_t)p0 * 4u + 16u, out_a + 4, out_r + 4);
      cur = nxt;
    }
    if (REWARD && sr.reward_sum != nullptr) {  // uniform: reward_sum is a kernel argument
      const double total = block_sum(rr.sum, lds_sum);
      if (threadIdx.x == 0) sr.reward_sum[b] = (float)total;
    }
  }
}

// ---------------------------------------------------------------- group normalisation
__global__ __launch_bounds__(kBlock) void scatter_kernel(const float* __restrict__ src,
                                                         const int64_t* __restrict__ indices, int64_t n,
                                                         float* __restrict__ dst) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t slot = indices ? indices[i] : i;
    if (slot >= 0 && slot < n) dst[slot] = src[i];
  }
}

__global__ __launch_bounds__(kBlock) void group_normalize_kernel(const float* __restrict__ ordered,
                                                                 const int64_t* __restrict__ indices, int64_t n_total,
                                                                 int64_t n_samples, int estimator,
                                                                 float* __restrict__ out,
                                                                 float* __restrict__ group_std) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_total; i += (int64_t)gridDim.x * kBlock) {
    const int64_t slot = indices ? indices[i] : i;
    if (slot < 0 || slot >= n_total) {
      out[i] = NAN;
      if (group_std) group_std[i] = NAN;
      continue;
    }
    const float* grp = ordered + (slot / n_samples) * n_samples;
    double sum = 0.0;
    for (int64_t k = 0; k < n_samples; ++k) sum += (double)grp[k];
    const double mean = sum / (double)n_samples;
    double ss = 0.0;
    for (int64_t k = 0; k < n_samples; ++k) {
      const double d = (double)grp[k] - mean;
      ss += d * d;
    }
    const double std_unbiased = sqrt(ss / (double)(n_samples - 1));  // NaN for n == 1, like torch.std
    const double x = (double)ordered[slot];
    double y = x;
    if (estimator == ORLHF_GROUP_RLOO)
      y = x - (sum - x) / (double)(n_samples - 1);
    else if (estimator == ORLHF_GROUP_BASELINE)
      y = x - mean;
    else if (estimator == ORLHF_GROUP_NORM)
      y = (x - mean) / (std_unbiased + 1e-9);
    out[i] = (float)y;
    if (group_std) group_std[i] = (float)std_unbiased;
  }
}

// ---------------------------------------------------------------- global masked whitening
constexpr int kWhitenBlocks = 1024;

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void whiten_partial_kernel(const float* __restrict__ x,
                                                                const void* __restrict__ mask, int64_t n,
                                                                double* __restrict__ partial) {
  __shared__ double lds[kWavesPerBlock];
  double sx = 0.0, sxx = 0.0, sm = 0.0;
  auto add = [&](float xv, float mv) {
    const double m = (double)mv, v = (double)xv;
    sx += v * m;
    sxx += v * v * m;
    sm += m;
  };
  const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x, stride = (int64_t)gridDim.x * kBlock;
  const int64_t groups = n / 4;
#pragma unroll 4
  for (int64_t g = first; g < groups; g += stride) {
    const f32x4 v = *(const f32x4e*)(x + g * 4);
    float m[4];
    load_mask4<MASK_DT>(mask, g * 4, m);
#pragma unroll
    for (int k = 0; k < 4; ++k) add(v[k], m[k]);
  }
  for (int64_t i = groups * 4 + first; i < n; i += stride) add(x[i], load_mask<MASK_DT>(mask, i));
  sx = block_sum(sx, lds);
  sxx = block_sum(sxx, lds);
  sm = block_sum(sm, lds);
  if (threadIdx.x == 0) {
    partial[blockIdx.x * 3 + 0] = sx;
    partial[blockIdx.x * 3 + 1] = sxx;
    partial[blockIdx.x * 3 + 2] = sm;
  }
}

// partial -> {mean, rstd} as floats right after the partials
__global__ __launch_bounds__(kBlock) void whiten_final_kernel(const double* __restrict__ partial, int n_partial,
                                                              int std_norm, float* __restrict__ mean_rstd,
                                                              float* __restrict__ stats_out) {
  __shared__ double lds[kWavesPerBlock];
  double sx = 0.0, sxx = 0.0, sm = 0.0;
  constexpr int kBatch = 8;  // entries per lane loaded together: one workgroup, latency-bound
  for (int i0 = threadIdx.x; i0 < n_partial; i0 += kBatch * kBlock) {
    double v[kBatch][3];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = i0 + u * kBlock;
#pragma unroll
      for (int q = 0; q < 3; ++q) v[u][q] = i < n_partial ? partial[(int64_t)i * 3 + q] : 0.0;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      sx += v[u][0];
      sxx += v[u][1];
      sm += v[u][2];
    }
  }
  sx = block_sum(sx, lds);
  sxx = block_sum(sxx, lds);
  sm = block_sum(sm, lds);
  if (threadIdx.x == 0) {
    const double mean = sx / sm;
    // sum((x-mean)^2 m)/sum(m) expanded; fp64 keeps the cancellation harmless
    double var = sxx / sm - mean * mean;
    double rstd = 1.0;
    if (std_norm) rstd = 1.0 / sqrt(var > 1e-8 ? var : (var != var ? var : 1e-8));
    mean_rstd[0] = (float)mean;
    mean_rstd[1] = (float)rstd;
    if (stats_out != nullptr) {
      stats_out[0] = (float)mean;
      stats_out[1] = (float)rstd;
    }
  }
}

// out may be x itself (each lane reads its elements before it writes them): no __restrict__ on them
__global__ __launch_bounds__(kBlock) void whiten_apply_kernel(const float* x, int64_t n,
                                                              const float* __restrict__ mean_rstd, float* out) {
  const float mean = mean_rstd[0], rstd = mean_rstd[1];
  const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x, stride = (int64_t)gridDim.x * kBlock;
  const int64_t groups = n / 4;
#pragma unroll 2
  for (int64_t g = first; g < groups; g += stride) {
    const f32x4 v = stream_load4(x + g * 4);
    f32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = (v[k] - mean) * rstd;
    *(f32x4e*)(out + g * 4) = o;
  }
  for (int64_t i = groups * 4 + first; i < n; i += stride) out[i] = (x[i] - mean) * rstd;
}

// ---- whitening over a list of blocks (one per experience) without gathering them first.
// A launch carries up to kSegs blocks in its arguments; a workgroup finds its block from the
// table of first workgroup indices and works on kWhitenSpan consecutive elements of it.
constexpr int kSegs = 16;
constexpr int kWhitenSpan = kBlock * 4 * 8;

struct WhitenSegs {
  const float* x[kSegs];
  const void* mask[kSegs];  // statistics pass
  float* out[kSegs];        // apply pass
  int64_t n[kSegs];
  int first_wg[kSegs + 1];
  int n_segs;
};

// Calls four(i0) / one(i) over the span of this workgroup inside its block.
template <typename F4, typename F1>
__device__ __forceinline__ void for_span(int64_t lo, int64_t hi, F4&& four, F1&& one) {
#pragma unroll 2
  for (int64_t s0 = lo; s0 < hi; s0 += kBlock * 4) {
    if (s0 + kBlock * 4 <= hi) {
      four(s0 + (int64_t)threadIdx.x * 4);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int64_t i = s0 + threadIdx.x + k * kBlock;
        if (i < hi) one(i);
      }
    }
  }
}

__device__ __forceinline__ int segment_of(const WhitenSegs& segs, int wg) {
  int s = 0;
  while (s + 1 < segs.n_segs && wg >= segs.first_wg[s + 1]) ++s;
  return s;
}

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void whiten_partial_multi_kernel(WhitenSegs segs, double* __restrict__ partial) {
  __shared__ double lds[kWavesPerBlock];
  const int s = segment_of(segs, blockIdx.x);
  const float* x = segs.x[s];
  const void* mask = segs.mask[s];
  const int64_t lo = (int64_t)(blockIdx.x - segs.first_wg[s]) * kWhitenSpan;
  const int64_t hi = lo + kWhitenSpan < segs.n[s] ? lo + kWhitenSpan : segs.n[s];
  double sx = 0.0, sxx = 0.0, sm = 0.0;
  auto add = [&](float xv, float mv) {
    const double m = (double)mv, v = (double)xv;
    sx += v * m;
    sxx += v * v * m;
    sm += m;
  };
  for_span(
      lo, hi,
      [&](int64_t i0) {
        const f32x4 v = *(const f32x4e*)(x + i0);
        float m[4];
        load_mask4<MASK_DT>(mask, i0, m);
#pragma unroll
        for (int k = 0; k < 4; ++k) add(v[k], m[k]);
      },
      [&](int64_t i) { add(x[i], load_mask<MASK_DT>(mask, i)); });
  sx = block_sum(sx, lds);
  sxx = block_sum(sxx, lds);
  sm = block_sum(sm, lds);
  if (threadIdx.x == 0) {
    partial[blockIdx.x * 3 + 0] = sx;
    partial[blockIdx.x * 3 + 1] = sxx;
    partial[blockIdx.x * 3 + 2] = sm;
  }
}

__global__ __launch_bounds__(kBlock) void whiten_apply_multi_kernel(WhitenSegs segs,
                                                                    const float* __restrict__ mean_rstd) {
  const int s = segment_of(segs, blockIdx.x);
  const float* x = segs.x[s];
  float* out = segs.out[s];
  const int64_t lo = (int64_t)(blockIdx.x - segs.first_wg[s]) * kWhitenSpan;
  const int64_t hi = lo + kWhitenSpan < segs.n[s] ? lo + kWhitenSpan : segs.n[s];
  const float mean = mean_rstd[0], rstd = mean_rstd[1];
  for_span(
      lo, hi,
      [&](int64_t i0) {
        const f32x4 v = stream_load4(x + i0);
        f32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = (v[k] - mean) * rstd;
        *(f32x4e*)(out + i0) = o;
      },
      [&](int64_t i) { out[i] = (x[i] - mean) * rstd; });
}

static inline int64_t span_wgs(int64_t n) { return (n + kWhitenSpan - 1) / kWhitenSpan; }

template <bool GAE, bool REWARD>
static void launch_scan(int mask_dtype, Rows rows, const float* values, const float* rewards, const void* mask,
                        double gamma, double coef, const SeqReward& sr, float* adv, float* ret, hipStream_t s) {
  const dim3 grid(slot_grid(row_slots(rows.n_rows), 65536)), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                        \
  hipLaunchKernelGGL((reverse_scan_kernel<M, GAE, REWARD>), grid, block, 0, s, rows, values, rewards, mask, gamma, \
                     coef, sr, adv, ret)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_compute_reward(const float* r, float kl_coef, const float* kl, const void* mask,
                                    int mask_dtype, int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens,
                                    int has_clip, float clip_low, float clip_high, float* reward,
                                    int64_t* eos_index, orlhf_stream_t stream) {
  if (int rc = check_rows("compute_reward", n_rows, n_cols, mask, mask_dtype)) return rc;
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(r && reward && (kl || n_cols == 0), "compute_reward: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  const Rows rows{n_rows, n_cols, cu_seqlens};
  const float neg_coef = -(kl_coef > 0.0f ? kl_coef : 0.0f);
  const dim3 grid(slot_grid(row_slots(n_rows), 65536)), block(kBlock);
#define ORLHF_LAUNCH(M)                                                                                         \
  hipLaunchKernelGGL(compute_reward_kernel<M>, grid, block, 0, s, rows, r, neg_coef, kl, mask, has_clip, clip_low, \
                     clip_high, reward, eos_index)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
  ORLHF_CHECK_LAUNCH("orlhf_compute_reward");
  return ORLHF_OK;
}

extern "C" int orlhf_gae_scan(const float* values, const float* rewards, const void* mask, int mask_dtype,
                              int64_t n_rows, int64_t n_cols, const int64_t* cu_seqlens, const int64_t* row_order,
                              float gamma, float lambd, float* advantages, float* returns, orlhf_stream_t stream) {
  if (int rc = check_rows("gae_scan", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(n_cols < (1ll << 30), "gae_scan: rows of %lld tokens (the limit is 2^30 - 1)", (long long)n_cols);
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(values && rewards && advantages && returns, "gae_scan: NULL pointer");
  const Rows rows{n_rows, n_cols, cu_seqlens, 0, row_order};
  launch_scan<true, false>(mask_dtype, rows, values, rewards, mask, (double)gamma, (double)gamma * (double)lambd,
                           SeqReward{}, advantages, returns, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_gae_scan");
  return ORLHF_OK;
}

extern "C" int orlhf_discounted_returns(const float* rewards, const void* mask, int mask_dtype, int64_t n_rows,
                                        int64_t n_cols, const int64_t* cu_seqlens, const int64_t* row_order,
                                        float gamma, float* returns, orlhf_stream_t stream) {
  if (int rc = check_rows("discounted_returns", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(n_cols < (1ll << 30), "discounted_returns: rows of %lld tokens (the limit is 2^30 - 1)", (long long)n_cols);
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(rewards && returns, "discounted_returns: NULL pointer");
  const Rows rows{n_rows, n_cols, cu_seqlens, 0, row_order};
  launch_scan<false, false>(mask_dtype, rows, nullptr, rewards, mask, (double)gamma, (double)gamma, SeqReward{},
                            nullptr, returns, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_discounted_returns");
  return ORLHF_OK;
}

extern "C" int orlhf_reward_scan(const float* r, float kl_coef, const float* kl, const float* values,
                                 const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                                 const int64_t* cu_seqlens, const int64_t* row_order, int has_clip, float clip_low,
                                 float clip_high, float gamma, float lambd, float* advantages, float* returns,
                                 float* reward_sum, orlhf_stream_t stream) {
  if (int rc = check_rows("reward_scan", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(n_cols < (1ll << 30), "reward_scan: rows of %lld tokens (the limit is 2^30 - 1)", (long long)n_cols);
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(r != nullptr && returns != nullptr && (kl != nullptr || n_cols == 0), "reward_scan: NULL pointer");
  ORLHF_CHECK_ARG((values == nullptr) == (advantages == nullptr),
                  "reward_scan: values and advantages go together (GAE) or are both NULL (discounted returns)");
  const Rows rows{n_rows, n_cols, cu_seqlens, 0, row_order};
  const SeqReward sr{r, -(kl_coef > 0.0f ? kl_coef : 0.0f), has_clip, clip_low, clip_high, reward_sum};
  if (values != nullptr)
    launch_scan<true, true>(mask_dtype, rows, values, kl, mask, (double)gamma, (double)gamma * (double)lambd, sr,
                            advantages, returns, (hipStream_t)stream);
  else
    launch_scan<false, true>(mask_dtype, rows, nullptr, kl, mask, (double)gamma, (double)gamma, sr, nullptr, returns,
                             (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_reward_scan");
  return ORLHF_OK;
}

extern "C" int orlhf_group_normalize(const float* rewards, const int64_t* indices, int64_t n_prompts,
                                     int64_t n_samples, int estimator, float* out, float* group_std,
                                     void* workspace, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_prompts >= 0 && n_samples >= 1, "group_normalize: n_prompts=%lld n_samples=%lld",
                  (long long)n_prompts, (long long)n_samples);
  ORLHF_CHECK_ARG(estimator >= ORLHF_GROUP_IDENTITY && estimator <= ORLHF_GROUP_NORM,
                  "group_normalize: unknown estimator %d", estimator);
  const int64_t n = n_prompts * n_samples;
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(rewards && out && workspace, "group_normalize: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  float* ordered = (float*)workspace;
  hipLaunchKernelGGL(scatter_kernel, dim3(flat_grid(n, 4096)), dim3(kBlock), 0, s, rewards, indices, n, ordered);
  ORLHF_CHECK_LAUNCH("orlhf_group_normalize(scatter)");
  hipLaunchKernelGGL(group_normalize_kernel, dim3(flat_grid(n, 4096)), dim3(kBlock), 0, s, ordered, indices, n,
                     n_samples, estimator, out, group_std);
  ORLHF_CHECK_LAUNCH("orlhf_group_normalize");
  return ORLHF_OK;
}

extern "C" int64_t orlhf_whiten_workspace_bytes(int64_t) {
  return (int64_t)kWhitenBlocks * 3 * (int64_t)sizeof(double) + 64;
}

extern "C" int64_t orlhf_whiten_multi_workspace_bytes(const int64_t* ns, int n_blocks) {
  int64_t wgs = 0;
  for (int i = 0; ns != nullptr && i < n_blocks; ++i) wgs += ns[i] > 0 ? span_wgs(ns[i]) : 0;
  return (wgs > 0 ? wgs : 1) * 3 * (int64_t)sizeof(double) + 64;
}

extern "C" int orlhf_masked_whiten_multi(const float* const* xs, const void* const* masks, int mask_dtype,
                                         const int64_t* ns, int n_blocks, int std_norm, void* workspace,
                                         float* const* outs, float* stats, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_blocks >= 0, "masked_whiten_multi: n_blocks=%d", n_blocks);
  ORLHF_CHECK_ARG(valid_mask_dtype(mask_dtype), "masked_whiten_multi: unknown mask dtype %d", mask_dtype);
  if (n_blocks == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(xs && ns && outs && workspace, "masked_whiten_multi: NULL pointer");
  ORLHF_CHECK_ARG(mask_dtype == ORLHF_MASK_NONE || masks != nullptr, "masked_whiten_multi: masks is NULL");
  int64_t total_wgs = 0;
  for (int i = 0; i < n_blocks; ++i) {
    ORLHF_CHECK_ARG(ns[i] >= 0, "masked_whiten_multi: ns[%d]=%lld", i, (long long)ns[i]);
    if (ns[i] == 0) continue;
    ORLHF_CHECK_ARG(xs[i] && outs[i], "masked_whiten_multi: block %d has a NULL pointer", i);
    ORLHF_CHECK_ARG(mask_dtype == ORLHF_MASK_NONE || masks[i] != nullptr, "masked_whiten_multi: mask %d is NULL", i);
    total_wgs += span_wgs(ns[i]);
  }
  if (total_wgs == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(total_wgs < (int64_t)1 << 30, "masked_whiten_multi: too many elements");
  hipStream_t s = (hipStream_t)stream;
  double* partial = (double*)workspace;
  float* mean_rstd = (float*)(partial + total_wgs * 3);
  const dim3 block(kBlock);
  // pass 0: statistics of every block into consecutive partial entries; pass 1: apply
  for (int pass = 0; pass < 2; ++pass) {
    int64_t done_wgs = 0;
    int i = 0;
    while (i < n_blocks) {
      WhitenSegs segs;
      segs.n_segs = 0;
      int wgs = 0;
      for (; i < n_blocks && segs.n_segs < kSegs; ++i) {
        if (ns[i] == 0) continue;
        const int k = segs.n_segs++;
        segs.x[k] = xs[i];
        segs.mask[k] = mask_dtype == ORLHF_MASK_NONE ? nullptr : masks[i];
        segs.out[k] = outs[i];
        segs.n[k] = ns[i];
        segs.first_wg[k] = wgs;
        wgs += (int)span_wgs(ns[i]);
      }
      if (segs.n_segs == 0) break;
      segs.first_wg[segs.n_segs] = wgs;
      if (pass == 0) {
        double* dst = partial + done_wgs * 3;
#define ORLHF_LAUNCH(M) hipLaunchKernelGGL(whiten_partial_multi_kernel<M>, dim3(wgs), block, 0, s, segs, dst)
        ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
        ORLHF_CHECK_LAUNCH("orlhf_masked_whiten_multi(partial)");
      } else {
        hipLaunchKernelGGL(whiten_apply_multi_kernel, dim3(wgs), block, 0, s, segs, mean_rstd);
        ORLHF_CHECK_LAUNCH("orlhf_masked_whiten_multi(apply)");
      }
      done_wgs += wgs;
    }
    if (pass == 0) {
      hipLaunchKernelGGL(whiten_final_kernel, dim3(1), block, 0, s, partial, (int)total_wgs, std_norm, mean_rstd, stats);
      ORLHF_CHECK_LAUNCH("orlhf_masked_whiten_multi(final)");
    }
  }
  return ORLHF_OK;
}

extern "C" int orlhf_masked_whiten(const float* x, const void* mask, int mask_dtype, int64_t n, int std_norm,
                                   void* workspace, float* out, float* stats, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0, "masked_whiten: n=%lld", (long long)n);
  ORLHF_CHECK_ARG(valid_mask_dtype(mask_dtype), "masked_whiten: unknown mask dtype %d", mask_dtype);
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(x && out && workspace, "masked_whiten: NULL pointer");
  ORLHF_CHECK_ARG(mask_dtype == ORLHF_MASK_NONE || mask != nullptr, "masked_whiten: mask is NULL");
  hipStream_t s = (hipStream_t)stream;
  double* partial = (double*)workspace;
  float* mean_rstd = (float*)(partial + (int64_t)kWhitenBlocks * 3);
  const int nb = flat_grid(n, kWhitenBlocks);
  const dim3 grid(nb), block(kBlock);
#define ORLHF_LAUNCH(M) hipLaunchKernelGGL(whiten_partial_kernel<M>, grid, block, 0, s, x, mask, n, partial)
  ORLHF_FOR_MASK_DTYPE(mask_dtype, ORLHF_LAUNCH)
#undef ORLHF_LAUNCH
  ORLHF_CHECK_LAUNCH("orlhf_masked_whiten(partial)");
  hipLaunchKernelGGL(whiten_final_kernel, dim3(1), block, 0, s, partial, nb, std_norm, mean_rstd, stats);
  ORLHF_CHECK_LAUNCH("orlhf_masked_whiten(final)");
  hipLaunchKernelGGL(whiten_apply_kernel, dim3(flat_grid((n + 3) / 4, 65536)), block, 0, s, x, n, mean_rstd, out);
  ORLHF_CHECK_LAUNCH("orlhf_masked_whiten(apply)");
  return ORLHF_OK;
}
