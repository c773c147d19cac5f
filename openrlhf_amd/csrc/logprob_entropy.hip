// Vocabulary-row kernels for gfx950: fused log-softmax + gather + entropy forward and its
// streaming backward. Both are pure HBM streams (read V elements per row; the backward also
// writes V elements), so the design goal is bytes in flight, not arithmetic:
//   * one 256-thread workgroup (4 wave64, one per SIMD) owns one vocabulary row;
//   * every lane issues ORLHF_ROW_UNROLL independent 16-byte loads before it touches the data
//     (8 x 4 KiB = 32 KiB per workgroup in flight with the default unroll);
//   * the softmax statistics are accumulated against a per-wave reference maximum taken from the
//     first 16-byte chunk of each lane instead of a running maximum: 1 fma + 1 v_exp_f32 + 2
//     accumulates per element. A row whose sums come out non-finite (an element more than ~88
//     nats above the reference, or inf/NaN logits) is re-read once with a classic per-lane online
//     maximum, so the result never depends on the shortcut;
//   * sums are kept in fp32 in 4 independent accumulators per lane, reduced over the wave with
//     cross-lane shuffles and over the 4 waves through LDS; the per-row epilogue runs in fp64;
//   * a launch with fewer rows than the chip has compute units cuts every row into segments, one
//     workgroup per (row, segment): the backward needs nothing else (an element's gradient depends
//     on the row only through its saved statistics), the forward writes one partial record per
//     segment, and a row's records are merged in a fixed order by the workgroup that finishes the
//     row's last segment (given a ticket per row) or by a small second kernel.
#include <stdlib.h>

#include "vocab_rows.h"

#ifndef ORLHF_ROW_UNROLL
#define ORLHF_ROW_UNROLL 8
#endif
#ifndef ORLHF_FWD_WAVES_PER_EU
#define ORLHF_FWD_WAVES_PER_EU 0
#endif

namespace orlhf {

// Visits every element of a row exactly once. f.vec(x, v) gets the kPerVec consecutive elements
// of body vector v (element index head + v*kPerVec); f.one(x, e) gets element e. With STORE the
// (modified) values are written to out_row at the same element positions in the same dtype.
// All in-row offsets are 32-bit: the row base stays in scalar registers.
template <int DT, bool STORE, typename F>
__device__ __forceinline__ void traverse_row(const char* row, char* out_row, const RowGeom& g,
                                             F& f) {
  using E = Elt<DT>;
  constexpr uint32_t U = ORLHF_ROW_UNROLL;
  constexpr uint32_t EPV = E::kPerVec;
  const uint32_t tid = threadIdx.x;
  const char* body = row + g.head * E::kSize;
  char* obody = STORE ? out_row + g.head * E::kSize : nullptr;

  const uint32_t nbatch = g.nvec / (kBlock * U);
  uint32_t v0 = tid;
  for (uint32_t b = 0; b < nbatch; ++b, v0 += kBlock * U) {
    u32x4 buf[U];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) buf[u] = load_vec(body + (v0 + u * kBlock) * 16u);
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      float x[EPV];
      E::unpack(buf[u], x);
      f.vec(x, v0 + u * kBlock);
      if (STORE) store_vec(obody + (v0 + u * kBlock) * 16u, E::pack(x));
    }
  }
  if (v0 < g.nvec) {  // last, partial batch: same loads in flight, predicated per vector
    u32x4 buf[U];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t v = v0 + u * kBlock;
      if (v < g.nvec) buf[u] = load_vec(body + v * 16u);
    }
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t v = v0 + u * kBlock;
      if (v < g.nvec) {
        float x[EPV];
        E::unpack(buf[u], x);
        f.vec(x, v);
        if (STORE) store_vec(obody + v * 16u, E::pack(x));
      }
    }
  }
  // scalar head + tail (at most 2*(kPerVec-1) elements unless scalar_only)
  const uint32_t nscalar = g.head + g.tail;
  for (uint32_t k = tid; k < nscalar; k += kBlock) {
    const uint32_t e = k < g.head ? k : g.head + g.nvec * EPV + (k - g.head);
    float x = E::load1(row + e * E::kSize);
    f.one(x, e);
    if (STORE) E::store1(out_row + e * E::kSize, x);
  }
}

constexpr int kAcc = 4;  // independent accumulators per lane

// Fast path: exponent = x*c - M with a wave-uniform reference M (no running maximum).
template <int MODE>
struct FastAcc {
  float cT, negMT, c1, negM1;
  float sT[kAcc], s1[kAcc], t1[kAcc];
  __device__ __forceinline__ void init(float m_ref, float c_scaled, float c_plain) {
    cT = c_scaled;
    c1 = c_plain;
    negMT = -(m_ref * c_scaled);
    negM1 = -(m_ref * c_plain);
#pragma unroll
    for (int k = 0; k < kAcc; ++k) sT[k] = s1[k] = t1[k] = 0.0f;
  }
  __device__ __forceinline__ void elem(float x, int k) {
    if (ModeTraits<MODE>::kScaledSet) sT[k] += fast_exp2(fmaf(x, cT, negMT));
    if (ModeTraits<MODE>::kPlainSet) {
      const float e = fast_exp2(fmaf(x, c1, negM1));
      s1[k] += e;
      t1[k] = fmaf(e, x, t1[k]);
    }
  }
  template <int N>
  __device__ __forceinline__ void vec(float (&x)[N], uint32_t) {
#pragma unroll
    for (int j = 0; j < N; ++j) elem(x[j], j % kAcc);
  }
  __device__ __forceinline__ void one(float& x, uint32_t) { elem(x, 0); }
  __device__ __forceinline__ void fold(float& st, float& s, float& t) const {
    st = (sT[0] + sT[1]) + (sT[2] + sT[3]);
    s = (s1[0] + s1[1]) + (s1[2] + s1[3]);
    t = (t1[0] + t1[1]) + (t1[2] + t1[3]);
  }
};

// Safe path: per-lane running maximum m (raw logit units), sums relative to it.
template <int MODE>
struct SafeAcc {
  float cT, c1;
  float m, sT, s1, t1;
  __device__ __forceinline__ void init(float c_scaled, float c_plain) {
    cT = c_scaled;
    c1 = c_plain;
    m = -INFINITY;
    sT = s1 = t1 = 0.0f;
  }
  __device__ __forceinline__ void raise(float cm) {
    if (cm > m) {  // also true for the first finite element (m == -inf)
      if (m != -INFINITY) {
        const float d = m - cm;  // < 0, or -inf when cm == +inf
        if (ModeTraits<MODE>::kScaledSet) sT *= fast_exp2(d * cT);
        if (ModeTraits<MODE>::kPlainSet) {
          const float r = fast_exp2(d * c1);
          s1 *= r;
          t1 *= r;
        }
      }
      m = cm;
    }
  }
  __device__ __forceinline__ void elem(float x) {
    if (m == -INFINITY) {
      // only -inf (or NaN) seen so far: exp() contributes 0 to the sums, but the reference's
      // softmax(x)*x is 0 * -inf = NaN for such an element (a NaN logit poisons everything).
      if (ModeTraits<MODE>::kPlainSet) t1 = NAN;
      if (x != x) sT = s1 = NAN;
      return;
    }
    // x == m covers m == +inf (inf - inf would be NaN): such an element counts as exp(0),
    // which makes logsumexp +inf and the entropy NaN, as in the reference
    const float d = (x == m) ? 0.0f : x - m;
    if (ModeTraits<MODE>::kScaledSet) sT += fast_exp2(d * cT);
    if (ModeTraits<MODE>::kPlainSet) {
      const float e = fast_exp2(d * c1);
      s1 += e;
      t1 = fmaf(e, x, t1);
    }
  }
  template <int N>
  __device__ __forceinline__ void vec(float (&x)[N], uint32_t) {
    float cm = x[0];
#pragma unroll
    for (int j = 1; j < N; ++j) cm = fmaxf(cm, x[j]);
    raise(cm);
#pragma unroll
    for (int j = 0; j < N; ++j) elem(x[j]);
  }
  __device__ __forceinline__ void one(float& x, uint32_t) {
    raise(x);
    elem(x);
  }
};

// Workgroup-combined sums. Fast pass: exponents were x*c - M, MT / M1 hold M (log2 units).
// Safe pass: exponents were (x - m)*c, MT and M1 both hold the row maximum m (logit units).
struct RowSums {
  float MT, sT, M1, s1, t1;
};

// How a launch cuts its rows: n segments of seg_elems elements (the last one shorter), work item
// w = row * n + segment. n == 1: whole rows. partials (forward only, n > 1): kPartial floats per
// work item {MT, sT, M1, s1, t1, fast-pass flag, the label's logit if it lies in the segment, 0}.
constexpr int kPartial = 8;
struct RowSplit {
  int n;
  uint32_t seg_elems;
  float* partials;
  int* tickets = nullptr;  // one per row, zero between launches: the segment that arrives last merges its row
};

struct WorkItem {
  int64_t row;
  uint32_t first;  // first element of the segment
  int64_t len;     // its length
};
__device__ __forceinline__ WorkItem work_item(int64_t w, const RowSplit& split, int64_t vocab) {
  if (split.n == 1) return {w, 0u, vocab};
  const int64_t row = w / split.n;
  const uint32_t first = (uint32_t)(w - row * split.n) * split.seg_elems;
  const int64_t left = vocab - first;
  return {row, first, left < (int64_t)split.seg_elems ? left : (int64_t)split.seg_elems};
}

__device__ __forceinline__ bool sums_usable(float s) { return s > 0.0f && s < INFINITY; }

// Merges the segment records of one row and finishes the row exactly as the whole-row epilogue
// does: ONE WAVE calls it, lane k holds segment k (at most 64), maxima and sums go through the
// fixed butterfly of the wave reductions in fp64, so the result does not depend on which segment was
// written when. FRESH: the records were written by other workgroups of the same launch; they are
// read past the L1, which may hold a line from before a neighbouring record was written.
template <bool FRESH>
__device__ __forceinline__ void merge_row(int64_t row_i, int64_t vocab, const int64_t* __restrict__ labels, double temperature,
                                          float* __restrict__ logprob, float* __restrict__ entropy,
                                          float* __restrict__ row_stats, bool scaled_set, bool plain_set, bool want_lp,
                                          const RowSplit& split) {
  const double c_plain = 1.4426950408889634, c_scaled = 1.4426950408889634 / temperature;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t label = want_lp ? labels[row_i] : -1;
  // maxima in log2 units: a fast-pass record holds them so, a safe-pass record holds the segment
  // maximum in logit units in both fields. Lanes past the last segment hold the neutral record.
  double mt = -INFINITY, m1 = -INFINITY, sT = 0.0, s1 = 0.0, t1 = 0.0;
  float x_label = 0.0f;  // the segment that holds the label has read its logit
  if (lane < split.n) {
    const float* rec = split.partials + (row_i * split.n + lane) * kPartial;
    float r[kPartial];
    if (FRESH) {
#pragma unroll
      for (int k = 0; k < kPartial; k += 2) {
        const uint64_t two = __hip_atomic_load((const uint64_t*)rec + k / 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        r[k] = as_float((uint32_t)two);
        r[k + 1] = as_float((uint32_t)(two >> 32));
      }
    } else {
      const f32x4 a = *(const f32x4*)rec, b = *(const f32x4*)(rec + 4);
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = a[k], r[4 + k] = b[k];
    }
    const bool fast = r[5] != 0.0f;
    mt = (double)r[0] * (fast ? 1.0 : c_scaled);
    m1 = (double)r[2] * (fast ? 1.0 : c_plain);
    sT = (double)r[1];
    s1 = (double)r[3];
    t1 = (double)r[4];
    if (label >= 0 && label < vocab && (uint32_t)lane == (uint32_t)label / split.seg_elems) x_label = r[6];
  }
  x_label = wave_sum(x_label);  // one lane holds it, the others 0
  double MT = mt, M1 = m1;
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const double ot = __shfl_xor(MT, o, kWave), o1 = __shfl_xor(M1, o, kWave);
    MT = ot > MT ? ot : MT;
    M1 = o1 > M1 ? o1 : M1;
  }
  // a segment at the row maximum (or one that saw nothing finite) keeps its sums as they are:
  // 0, or the NaN markers of the safe pass
  const double rT = (mt != -INFINITY && mt != MT) ? exp2(mt - MT) : 1.0;
  const double r1 = (m1 != -INFINITY && m1 != M1) ? exp2(m1 - M1) : 1.0;
  sT = wave_sum(sT * rT);
  s1 = wave_sum(s1 * r1);
  t1 = wave_sum(t1 * r1);
  if (lane != 0) return;
  double lse_t = 0.0, lse_1 = 0.0, ex = 0.0;
  if (scaled_set) lse_t = MT * kLn2d + log(sT);
  if (plain_set) {
    lse_1 = M1 * kLn2d + log(s1);
    ex = t1 / s1;
    if (!scaled_set) lse_t = lse_1;
  }
  if (want_lp) {
    float lp;
    if (label >= 0 && label < vocab) {
      lp = (float)((double)x_label / temperature - lse_t);
    } else {
      lp = (label == -100) ? 0.0f : NAN;
    }
    logprob[row_i] = lp;
  }
  if (plain_set && entropy != nullptr) entropy[row_i] = (float)(lse_1 - ex);
  if (row_stats != nullptr)
    *(f32x4*)(row_stats + row_i * 4) = f32x4{(float)lse_t, (float)(plain_set ? lse_1 : lse_t), (float)ex, 0.0f};
}

// ---------------------------------------------------------------- forward kernel
template <int DT, int MODE>
__global__ __launch_bounds__(kBlock) void logprob_entropy_fwd_kernel(
    const char* __restrict__ logits, int64_t n_rows, int64_t vocab, int64_t row_stride_bytes,
    const int64_t* __restrict__ labels, double temperature, float* __restrict__ logprob,
    float* __restrict__ entropy, float* __restrict__ row_stats, const uint8_t* __restrict__ row_mask,
    int scalar_only, RowSplit split) {
  using E = Elt<DT>;
  using MT = ModeTraits<MODE>;
  __shared__ float lds[kWavesPerBlock][8];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const float c_plain = kLog2e;
  const float c_scaled = (float)(1.4426950408889634 / temperature);

  const int64_t n_work = n_rows * split.n;
  for (int64_t work = blockIdx.x; work < n_work; work += gridDim.x) {
    const WorkItem item = work_item(work, split, vocab);
    const int64_t row_i = item.row;
    if (row_mask != nullptr && row_mask[row_i] == 0) {  // row not wanted: outputs 0, logits not read
      // cut rows: the merging kernel writes the zeros, or the row's first segment where nothing merges
      if (split.n > 1 && (split.tickets == nullptr || item.first != 0u)) continue;
      if (tid == 0) {
        if (MODE != kEntOnly && logprob != nullptr) logprob[row_i] = 0.0f;
        if (MT::kPlainSet && entropy != nullptr) entropy[row_i] = 0.0f;
        if (row_stats != nullptr) *(f32x4*)(row_stats + row_i * 4) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      }
      continue;
    }
    const char* row = logits + row_i * row_stride_bytes + (int64_t)item.first * E::kSize;
    const int64_t seg_len = item.len;
    const RowGeom g = row_geom<DT>(row, seg_len, scalar_only != 0);

    // the label and its logit, asked for now: the row's last instructions do not wait on two
    // dependent loads then (on a launch of a few microseconds that wait is a tenth of the whole)
    int64_t label = -1;
    float x_label = 0.0f;
    if (MODE != kEntOnly && logprob != nullptr && tid == 0) {
      label = labels[row_i];
      const int64_t at = label - (int64_t)item.first;
      if (at >= 0 && at < seg_len) x_label = E::load1(row + at * E::kSize);
    }

    // ---- reference maximum of this wave: first vector (or first scalar) of each lane
    float m_ref = -INFINITY;
    if (g.nvec > 0) {
      const uint32_t v = (uint32_t)tid < g.nvec ? (uint32_t)tid : g.nvec - 1;
      float x[E::kPerVec];
      // temporal load on purpose: the streaming pass reads these 4 KiB again and should hit in L2
      E::unpack(*(const u32x4*)(row + g.head * E::kSize + v * 16u), x);
#pragma unroll
      for (int j = 0; j < E::kPerVec; ++j) m_ref = fmaxf(m_ref, x[j]);
    } else {
      const uint32_t e = (uint32_t)tid < (uint32_t)seg_len ? (uint32_t)tid : (uint32_t)seg_len - 1;
      m_ref = E::load1(row + e * E::kSize);
    }
    m_ref = wave_max(m_ref);

    // ---- fast pass
    RowSums sums;
    {
      FastAcc<MODE> acc;
      acc.init(m_ref, c_scaled, c_plain);
      traverse_row<DT, false>(row, nullptr, g, acc);
      float st, s, t;
      acc.fold(st, s, t);
      st = wave_sum(st);
      s = wave_sum(s);
      t = wave_sum(t);
      if (lane == 0) {
        lds[wave][0] = -acc.negMT;
        lds[wave][1] = st;
        lds[wave][2] = -acc.negM1;
        lds[wave][3] = s;
        lds[wave][4] = t;
      }
      __syncthreads();
      float MTm = lds[0][0], M1m = lds[0][2];
#pragma unroll
      for (int w = 1; w < kWavesPerBlock; ++w) {
        MTm = fmaxf(MTm, lds[w][0]);
        M1m = fmaxf(M1m, lds[w][2]);
      }
      sums.MT = MTm;
      sums.M1 = M1m;
      sums.sT = sums.s1 = sums.t1 = 0.0f;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        const float rT = fast_exp2(lds[w][0] - MTm);
        const float r1 = fast_exp2(lds[w][2] - M1m);
        sums.sT = fmaf(lds[w][1], rT, sums.sT);
        sums.s1 = fmaf(lds[w][3], r1, sums.s1);
        sums.t1 = fmaf(lds[w][4], r1, sums.t1);
      }
      __syncthreads();
    }
    bool ok = true;
    if (MT::kScaledSet) ok = ok && sums_usable(sums.sT);
    if (MT::kPlainSet) ok = ok && sums_usable(sums.s1) && (fabsf(sums.t1) < INFINITY);

    // ---- safe pass (workgroup-uniform branch; rare)
    if (!ok) {
      SafeAcc<MODE> acc;
      acc.init(c_scaled, c_plain);
      traverse_row<DT, false>(row, nullptr, g, acc);
      const float m_w = wave_max(acc.m);
      // rescale each lane to the wave maximum; a lane that saw nothing finite keeps its
      // sums (0 or NaN markers) untouched
      float st = acc.sT, s = acc.s1, t = acc.t1;
      if (acc.m != -INFINITY && m_w != acc.m) {
        const float d = acc.m - m_w;
        st *= fast_exp2(d * c_scaled);
        const float r = fast_exp2(d * c_plain);
        s *= r;
        t *= r;
      }
      st = wave_sum(st);
      s = wave_sum(s);
      t = wave_sum(t);
      if (lane == 0) {
        lds[wave][0] = m_w;
        lds[wave][1] = st;
        lds[wave][3] = s;
        lds[wave][4] = t;
      }
      __syncthreads();
      float m_all = lds[0][0];
#pragma unroll
      for (int w = 1; w < kWavesPerBlock; ++w) m_all = fmaxf(m_all, lds[w][0]);
      sums.sT = sums.s1 = sums.t1 = 0.0f;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        const float mw = lds[w][0];
        float rT = 1.0f, r1 = 1.0f;
        if (mw != -INFINITY && mw != m_all) {
          rT = fast_exp2((mw - m_all) * c_scaled);
          r1 = fast_exp2((mw - m_all) * c_plain);
        }
        sums.sT += lds[w][1] * rT;
        sums.s1 += lds[w][3] * r1;
        sums.t1 += lds[w][4] * r1;
      }
      sums.MT = sums.M1 = m_all;
      __syncthreads();
    }

    if (split.n > 1) {  // a segment: its sums go to the merging kernel as they are
      int drawn = 0;
      if (tid == 0) {
        float* rec = split.partials + work * kPartial;
        const float r[kPartial] = {sums.MT, sums.sT, sums.M1, sums.s1, sums.t1, ok ? 1.0f : 0.0f, x_label, 0.0f};
        if (split.tickets == nullptr) {
          *(f32x4*)rec = f32x4{r[0], r[1], r[2], r[3]};
          *(f32x4*)(rec + 4) = f32x4{r[4], r[5], r[6], r[7]};
        } else {
          // The segment that takes the row's last ticket finds every record of the row written and
          // merges them, in segment order whoever came when. Nobody waits for anybody; the ticket
          // goes back to zero for the next launch. Records and tickets go to and come from device
          // memory as device-scope accesses, which pass the caches that the compute dies do not
          // share; a writer has its stores acknowledged before it draws. (A device-scope fence
          // would do as well, at the price of walking a die's whole L2 per workgroup: several
          // microseconds on a launch that takes ten.)
#pragma unroll
          for (int k = 0; k < kPartial; k += 2) {
            const uint64_t two = (uint64_t)__builtin_bit_cast(uint32_t, r[k]) | (uint64_t)__builtin_bit_cast(uint32_t, r[k + 1]) << 32;
            __hip_atomic_store((uint64_t*)rec + k / 2, two, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this thread's stores have been acknowledged
          drawn = __hip_atomic_fetch_add(split.tickets + row_i, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      if (split.tickets != nullptr && wave == 0) {  // the other waves go on to their next segment
        if (__shfl(drawn, 0, kWave) == split.n - 1) {
          merge_row<true>(row_i, vocab, labels, temperature, logprob, entropy, row_stats, MT::kScaledSet, MT::kPlainSet,
                          MODE != kEntOnly && logprob != nullptr, split);
          if (lane == 0) __hip_atomic_store(split.tickets + row_i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      continue;
    }

    // ---- per-row epilogue in fp64
    if (tid == 0) {
      double lse_t = 0.0, lse_1 = 0.0, ex = 0.0;
      if (MT::kScaledSet) {
        const double base = ok ? (double)sums.MT * kLn2d : (double)sums.MT / temperature;
        lse_t = base + log((double)sums.sT);
      }
      if (MT::kPlainSet) {
        const double base = ok ? (double)sums.M1 * kLn2d : (double)sums.M1;
        lse_1 = base + log((double)sums.s1);
        ex = (double)sums.t1 / (double)sums.s1;
        if (!MT::kScaledSet) lse_t = lse_1;  // T == 1 (or entropy only)
      }
      if (MODE != kEntOnly && logprob != nullptr) {
        float lp;
        if (label >= 0 && label < vocab) {
          lp = (float)((double)x_label / temperature - lse_t);
        } else {
          lp = (label == -100) ? 0.0f : NAN;
        }
        logprob[row_i] = lp;
      }
      if (MT::kPlainSet && entropy != nullptr) entropy[row_i] = (float)(lse_1 - ex);
      if (row_stats != nullptr) {
        f32x4 st = {(float)lse_t, (float)(MT::kPlainSet ? lse_1 : lse_t), (float)ex, 0.0f};
        *(f32x4*)(row_stats + row_i * 4) = st;
      }
    }
  }
}

// The merge as a launch of its own (callers that pass no tickets): one wave per row.
template <int DT>
__global__ __launch_bounds__(kBlock) void logprob_entropy_merge_kernel(
    int64_t n_rows, int64_t vocab, const int64_t* __restrict__ labels, double temperature, float* __restrict__ logprob,
    float* __restrict__ entropy, float* __restrict__ row_stats, const uint8_t* __restrict__ row_mask,
    int mode, RowSplit split) {
  const bool scaled_set = (mode == kLpOnly || mode == kBothT), plain_set = (mode != kLpOnly);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row_i = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row_i >= n_rows) return;
  const bool want_lp = mode != kEntOnly && logprob != nullptr;
  if (row_mask != nullptr && row_mask[row_i] == 0) {
    if (lane == 0) {
      if (want_lp) logprob[row_i] = 0.0f;
      if (plain_set && entropy != nullptr) entropy[row_i] = 0.0f;
      if (row_stats != nullptr) *(f32x4*)(row_stats + row_i * 4) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    return;
  }
  merge_row<false>(row_i, vocab, labels, temperature, logprob, entropy, row_stats, scaled_set, plain_set, want_lp, split);
}

// ---------------------------------------------------------------- backward kernel
// Zero-fills a row without reading it.
template <int DT>
__device__ __forceinline__ void zero_row(char* out_row, const RowGeom& g) {
  using E = Elt<DT>;
  const uint32_t tid = threadIdx.x;
  char* obody = out_row + g.head * E::kSize;
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (uint32_t v = tid; v < g.nvec; v += kBlock) store_vec(obody + v * 16u, z);
  const uint32_t nscalar = g.head + g.tail;
  for (uint32_t k = tid; k < nscalar; k += kBlock) {
    const uint32_t e = k < g.head ? k : g.head + g.nvec * E::kPerVec + (k - g.head);
    E::store1(out_row + e * E::kSize, 0.0f);
  }
}

template <int DT, int MODE>
__global__ __launch_bounds__(kBlock) void logprob_entropy_bwd_kernel(
    const char* logits, char* grad, int64_t n_rows, int64_t vocab, int64_t row_stride_bytes,
    int64_t grad_stride_bytes, const int64_t* __restrict__ labels, double temperature,
    const float* __restrict__ g_logprob, const float* __restrict__ g_entropy,
    const float* __restrict__ row_stats, const uint8_t* __restrict__ row_mask, int scalar_only,
    RowSplit split) {
  const double inv_t = 1.0 / temperature;
  const int64_t n_work = n_rows * split.n;
  for (int64_t work = blockIdx.x; work < n_work; work += gridDim.x) {
    const WorkItem item = work_item(work, split, vocab);
    const int64_t row_i = item.row;
    const char* row = logits + row_i * row_stride_bytes + (int64_t)item.first * Elt<DT>::kSize;
    char* out_row = grad + row_i * grad_stride_bytes + (int64_t)item.first * Elt<DT>::kSize;
    // the geometry follows the OUTPUT row when only zeros are written, the input row otherwise
    // (the host guarantees both have the same 16-byte phase unless scalar_only is set)
    const RowGeom g = row_geom<DT>(row, item.len, scalar_only != 0);

    const float glp = (MODE != kBwdEnt) ? g_logprob[row_i] : 0.0f;
    const float gh = (MODE != kBwdLp) ? g_entropy[row_i] : 0.0f;
    const bool skipped = row_mask != nullptr && row_mask[row_i] == 0;  // forward gave constants
    if (skipped || (glp == 0.0f && gh == 0.0f)) {
      zero_row<DT>(out_row, g);
      continue;
    }
    const f32x4 st = *(const f32x4*)(row_stats + row_i * 4);
    GradFn<MODE> fn;
    fn.cT = (float)(1.4426950408889634 * inv_t);
    fn.c1 = kLog2e;
    fn.negLT = -(float)((double)st[0] * 1.4426950408889634);
    fn.negL1 = -(float)((double)st[1] * 1.4426950408889634);
    fn.a_lp = -(float)((double)glp * inv_t);
    fn.onehot = (float)((double)glp * inv_t);
    fn.gh = gh;
    fn.k1 = gh * st[2] - (MODE == kBwdBothT1 ? glp : 0.0f);
    // the label relative to this segment; outside it (or outside the vocabulary) no element gets the one-hot term
    const int64_t label = (MODE != kBwdEnt) ? labels[row_i] : -1;
    fn.set_label((label >= 0 && label < vocab) ? label - (int64_t)item.first : -1, item.len, g, Elt<DT>::kPerVec);
    traverse_row<DT, true>(row, out_row, g, fn);
  }
}

// ---------------------------------------------------------------- host side
static int grid_for_rows(int64_t n_rows) {
  // one workgroup per row; cap the grid and stride over rows beyond it
  const int64_t cap = 1 << 20;
  return (int)(n_rows < cap ? n_rows : cap);
}

// Rows are cut when there are fewer of them than compute units: enough segments for about two
// workgroups per CU of a 256-CU part, none shorter than 32 KiB (one full batch of loads per lane),
// at most 64. Segment lengths are multiples of 16 elements so every segment keeps its row's
// 16-byte phase. The rule depends on the shape only, so results do not depend on the device.
static RowSplit row_split(int64_t n_rows, int64_t vocab, int esize) {
  RowSplit split{1, (uint32_t)vocab, nullptr};
  constexpr int64_t kWholeRowsFrom = 256, kItems = 512, kMinSegBytes = 32768, kMaxSplit = 64;
  if (n_rows >= kWholeRowsFrom) return split;
  int64_t n = (kItems + n_rows - 1) / n_rows;
  if (n > kMaxSplit) n = kMaxSplit;
  if (n > vocab * esize / kMinSegBytes) n = vocab * esize / kMinSegBytes;
  if (n <= 1) return split;
  const int64_t seg = (((vocab + n - 1) / n) + 15) & ~(int64_t)15;
  split.n = (int)((vocab + seg - 1) / seg);
  split.seg_elems = (uint32_t)seg;
  return split;
}

template <int DT>
static int launch_fwd(const void* logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                      const int64_t* labels, double temperature, float* logprob, float* entropy,
                      float* row_stats, const uint8_t* row_mask, void* workspace, int64_t workspace_bytes, int* tickets,
                      hipStream_t stream) {
  using E = Elt<DT>;
  const bool want_lp = logprob != nullptr;
  const bool want_ent = entropy != nullptr;
  const bool t1 = (temperature == 1.0);
  const int mode = !want_ent ? kLpOnly : (!want_lp ? kEntOnly : (t1 ? kBothT1 : kBothT));
  const char* p = (const char*)logits;
  const int64_t stride_bytes = row_stride * E::kSize;
  const int scalar_only = 0;
  RowSplit split{1, (uint32_t)vocab, nullptr};
  if (workspace != nullptr) {  // the caller offers room for segment records
    split = row_split(n_rows, vocab, E::kSize);
    if (split.n > 1) {
      ORLHF_CHECK_ARG(workspace_bytes >= n_rows * split.n * kPartial * (int64_t)sizeof(float) &&
                          ((uintptr_t)workspace & 15u) == 0,
                      "logprob_entropy_fwd_split: workspace of %lld bytes too small or not 16-byte aligned",
                      (long long)workspace_bytes);
      split.partials = (float*)workspace;
      split.tickets = tickets;
    }
  }
  const dim3 grid(grid_for_rows(n_rows * split.n)), block(kBlock);
#define ORLHF_FWD(M)                                                                          \
  hipLaunchKernelGGL((logprob_entropy_fwd_kernel<DT, M>), grid, block, 0, stream, p, n_rows,  \
                     vocab, stride_bytes, labels, temperature, logprob, entropy, row_stats,   \
                     row_mask, scalar_only, split)
  switch (mode) {
    case kLpOnly: ORLHF_FWD(kLpOnly); break;
    case kEntOnly: ORLHF_FWD(kEntOnly); break;
    case kBothT1: ORLHF_FWD(kBothT1); break;
    default: ORLHF_FWD(kBothT); break;
  }
#undef ORLHF_FWD
  ORLHF_CHECK_LAUNCH("orlhf_logprob_entropy_fwd");
  if (split.n > 1 && split.tickets == nullptr) {
    hipLaunchKernelGGL((logprob_entropy_merge_kernel<DT>), dim3((unsigned)((n_rows + kWavesPerBlock - 1) / kWavesPerBlock)), block, 0,
                       stream, n_rows, vocab, labels, temperature, logprob, entropy, row_stats, row_mask, mode, split);
    ORLHF_CHECK_LAUNCH("orlhf_logprob_entropy_fwd_split(merge)");
  }
  return ORLHF_OK;
}

template <int DT>
static int launch_bwd(const void* logits, void* grad, int64_t n_rows, int64_t vocab,
                      int64_t row_stride, int64_t grad_row_stride, const int64_t* labels,
                      double temperature, const float* g_logprob, const float* g_entropy,
                      const float* row_stats, const uint8_t* row_mask, hipStream_t stream) {
  using E = Elt<DT>;
  const bool has_lp = g_logprob != nullptr;
  const bool has_ent = g_entropy != nullptr;
  const bool t1 = (temperature == 1.0);
  const int mode = !has_ent ? kBwdLp : (!has_lp ? kBwdEnt : (t1 ? kBwdBothT1 : kBwdBothT));
  const char* p = (const char*)logits;
  char* gp = (char*)grad;
  const int64_t stride_bytes = row_stride * E::kSize;
  const int64_t gstride_bytes = grad_row_stride * E::kSize;
  // vector path needs input and output rows on the same 16-byte phase
  const bool same_phase = (((uintptr_t)p ^ (uintptr_t)gp) & 15u) == 0 &&
                          ((stride_bytes - gstride_bytes) & 15) == 0;
  const int scalar_only = same_phase ? 0 : 1;
  const RowSplit split = row_split(n_rows, vocab, E::kSize);
  const dim3 grid(grid_for_rows(n_rows * split.n)), block(kBlock);
#define ORLHF_BWD(M)                                                                          \
  hipLaunchKernelGGL((logprob_entropy_bwd_kernel<DT, M>), grid, block, 0, stream, p, gp,      \
                     n_rows, vocab, stride_bytes, gstride_bytes, labels, temperature,         \
                     g_logprob, g_entropy, row_stats, row_mask, scalar_only, split)
  switch (mode) {
    case kBwdLp: ORLHF_BWD(kBwdLp); break;
    case kBwdEnt: ORLHF_BWD(kBwdEnt); break;
    case kBwdBothT1: ORLHF_BWD(kBwdBothT1); break;
    default: ORLHF_BWD(kBwdBothT); break;
  }
#undef ORLHF_BWD
  ORLHF_CHECK_LAUNCH("orlhf_logprob_entropy_bwd");
  return ORLHF_OK;
}

// logits <- round_to_dtype(logits / divisor), row by row: the reference's in-place
// logits.div_(temperature) for callers that rely on that side effect.
struct DivideFn {
  float divisor;
  template <int N>
  __device__ __forceinline__ void vec(float (&x)[N], uint32_t) const {
#pragma unroll
    for (int j = 0; j < N; ++j) x[j] = x[j] / divisor;
  }
  __device__ __forceinline__ void one(float& x, uint32_t) const { x = x / divisor; }
};

template <int DT>
__global__ __launch_bounds__(kBlock) void divide_rows_kernel(char* logits, int64_t n_rows, int64_t vocab,
                                                             int64_t row_stride_bytes, float divisor) {
  DivideFn fn{divisor};
  for (int64_t row_i = blockIdx.x; row_i < n_rows; row_i += gridDim.x) {
    char* row = logits + row_i * row_stride_bytes;
    const RowGeom g = row_geom<DT>(row, vocab, false);
    traverse_row<DT, true>(row, row, g, fn);
  }
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_divide_rows_inplace(void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                         int64_t row_stride, double divisor, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && vocab > 0 && row_stride >= vocab, "divide_rows_inplace: n_rows=%lld vocab=%lld stride=%lld",
                  (long long)n_rows, (long long)vocab, (long long)row_stride);
  ORLHF_CHECK_ARG(vocab < (1ll << 29), "divide_rows_inplace: vocab %lld too large", (long long)vocab);
  ORLHF_CHECK_ARG(divisor == divisor && divisor != 0.0, "divide_rows_inplace: divisor must be a non-zero number");
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(logits != nullptr, "divide_rows_inplace: logits is NULL");
  const dim3 grid(grid_for_rows(n_rows)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  char* p = (char*)logits;
  switch (dtype) {
    case ORLHF_F32: hipLaunchKernelGGL(divide_rows_kernel<ORLHF_F32>, grid, block, 0, s, p, n_rows, vocab, row_stride * 4, (float)divisor); break;
    case ORLHF_BF16: hipLaunchKernelGGL(divide_rows_kernel<ORLHF_BF16>, grid, block, 0, s, p, n_rows, vocab, row_stride * 2, (float)divisor); break;
    case ORLHF_F16: hipLaunchKernelGGL(divide_rows_kernel<ORLHF_F16>, grid, block, 0, s, p, n_rows, vocab, row_stride * 2, (float)divisor); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "divide_rows_inplace: unknown dtype %d", dtype);
  }
  ORLHF_CHECK_LAUNCH("orlhf_divide_rows_inplace");
  return ORLHF_OK;
}

static int forward_entry(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                         const int64_t* labels, double temperature, float* logprob, float* entropy,
                         float* row_stats, const uint8_t* row_mask, int flags, void* workspace,
                         int64_t workspace_bytes, int32_t* tickets, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && vocab > 0, "logprob_entropy_fwd: n_rows=%lld vocab=%lld",
                  (long long)n_rows, (long long)vocab);
  ORLHF_CHECK_ARG(row_stride >= vocab, "logprob_entropy_fwd: row_stride %lld < vocab %lld",
                  (long long)row_stride, (long long)vocab);
  ORLHF_CHECK_ARG(vocab < (1ll << 29), "logprob_entropy_fwd: vocab %lld too large (row must stay below 2 GiB)",
                  (long long)vocab);
  ORLHF_CHECK_ARG(temperature > 0.0 && temperature == temperature,
                  "logprob_entropy_fwd: temperature must be > 0");
  ORLHF_CHECK_ARG(flags == 0, "logprob_entropy_fwd: unknown flags 0x%x", flags);
  if (n_rows == 0) return ORLHF_OK;  // nothing to launch; empty outputs may well be NULL
  ORLHF_CHECK_ARG(logprob != nullptr || entropy != nullptr,
                  "logprob_entropy_fwd: logprob and entropy are both NULL");
  ORLHF_CHECK_ARG(logits != nullptr, "logprob_entropy_fwd: logits is NULL");
  ORLHF_CHECK_ARG(logprob == nullptr || labels != nullptr, "logprob_entropy_fwd: labels is NULL");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case ORLHF_F32:
      ORLHF_CHECK_ARG(((uintptr_t)logits & 3u) == 0, "logprob_entropy_fwd: logits not 4-byte aligned");
      return launch_fwd<ORLHF_F32>(logits, n_rows, vocab, row_stride, labels, temperature, logprob,
                                   entropy, row_stats, row_mask, workspace, workspace_bytes, tickets, s);
    case ORLHF_BF16:
      ORLHF_CHECK_ARG(((uintptr_t)logits & 1u) == 0, "logprob_entropy_fwd: logits not 2-byte aligned");
      return launch_fwd<ORLHF_BF16>(logits, n_rows, vocab, row_stride, labels, temperature, logprob,
                                    entropy, row_stats, row_mask, workspace, workspace_bytes, tickets, s);
    case ORLHF_F16:
      ORLHF_CHECK_ARG(((uintptr_t)logits & 1u) == 0, "logprob_entropy_fwd: logits not 2-byte aligned");
      return launch_fwd<ORLHF_F16>(logits, n_rows, vocab, row_stride, labels, temperature, logprob,
                                   entropy, row_stats, row_mask, workspace, workspace_bytes, tickets, s);
    default:
      return fail(ORLHF_ERR_INVALID_ARG, "logprob_entropy_fwd: unknown dtype %d", dtype);
  }
}

extern "C" int orlhf_logprob_entropy_fwd(const void* logits, int dtype, int64_t n_rows,
                                         int64_t vocab, int64_t row_stride, const int64_t* labels,
                                         double temperature, float* logprob, float* entropy,
                                         float* row_stats, const uint8_t* row_mask, int flags,
                                         orlhf_stream_t stream) {
  return forward_entry(logits, dtype, n_rows, vocab, row_stride, labels, temperature, logprob, entropy, row_stats,
                       row_mask, flags, nullptr, 0, nullptr, stream);
}

extern "C" int64_t orlhf_logprob_entropy_split_workspace_bytes(int dtype, int64_t n_rows, int64_t vocab) {
  if (n_rows <= 0 || vocab <= 0 || vocab >= (1ll << 29)) return 0;
  const RowSplit split = row_split(n_rows, vocab, dtype == ORLHF_F32 ? 4 : 2);
  return split.n > 1 ? n_rows * split.n * kPartial * (int64_t)sizeof(float) : 0;
}

extern "C" int orlhf_logprob_entropy_fwd_split(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                               int64_t row_stride, const int64_t* labels, double temperature,
                                               float* logprob, float* entropy, float* row_stats,
                                               const uint8_t* row_mask, void* workspace, int64_t workspace_bytes,
                                               int32_t* tickets, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(((uintptr_t)tickets & 3u) == 0, "logprob_entropy_fwd_split: tickets not 4-byte aligned");
  ORLHF_CHECK_ARG(workspace != nullptr || orlhf_logprob_entropy_split_workspace_bytes(dtype, n_rows, vocab) == 0,
                  "logprob_entropy_fwd_split: this shape needs a workspace (orlhf_logprob_entropy_split_workspace_bytes)");
  return forward_entry(logits, dtype, n_rows, vocab, row_stride, labels, temperature, logprob, entropy, row_stats,
                       row_mask, 0, workspace, workspace_bytes, tickets, stream);
}

extern "C" int orlhf_logprob_entropy_bwd(const void* logits, void* grad_logits, int dtype,
                                         int64_t n_rows, int64_t vocab, int64_t row_stride,
                                         int64_t grad_row_stride, const int64_t* labels,
                                         double temperature, const float* g_logprob,
                                         const float* g_entropy, const float* row_stats,
                                         const uint8_t* row_mask, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && vocab > 0, "logprob_entropy_bwd: n_rows=%lld vocab=%lld",
                  (long long)n_rows, (long long)vocab);
  ORLHF_CHECK_ARG(row_stride >= vocab && grad_row_stride >= vocab,
                  "logprob_entropy_bwd: row strides %lld/%lld < vocab %lld", (long long)row_stride,
                  (long long)grad_row_stride, (long long)vocab);
  ORLHF_CHECK_ARG(vocab < (1ll << 29), "logprob_entropy_bwd: vocab %lld too large (row must stay below 2 GiB)",
                  (long long)vocab);
  ORLHF_CHECK_ARG(temperature > 0.0 && temperature == temperature,
                  "logprob_entropy_bwd: temperature must be > 0");
  if (n_rows == 0) return ORLHF_OK;  // nothing to launch; empty arrays may well be NULL
  ORLHF_CHECK_ARG(g_logprob != nullptr || g_entropy != nullptr,
                  "logprob_entropy_bwd: g_logprob and g_entropy are both NULL");
  ORLHF_CHECK_ARG(logits != nullptr && grad_logits != nullptr && row_stats != nullptr,
                  "logprob_entropy_bwd: NULL logits / grad_logits / row_stats");
  ORLHF_CHECK_ARG(g_logprob == nullptr || labels != nullptr, "logprob_entropy_bwd: labels is NULL");
  hipStream_t s = (hipStream_t)stream;
  const int esize = dtype == ORLHF_F32 ? 4 : 2;
  ORLHF_CHECK_ARG((((uintptr_t)logits | (uintptr_t)grad_logits) & (uintptr_t)(esize - 1)) == 0,
                  "logprob_entropy_bwd: pointers not aligned to the element size");
  switch (dtype) {
    case ORLHF_F32:
      return launch_bwd<ORLHF_F32>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride,
                                   labels, temperature, g_logprob, g_entropy, row_stats, row_mask, s);
    case ORLHF_BF16:
      return launch_bwd<ORLHF_BF16>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride,
                                    labels, temperature, g_logprob, g_entropy, row_stats, row_mask, s);
    case ORLHF_F16:
      return launch_bwd<ORLHF_F16>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride,
                                   labels, temperature, g_logprob, g_entropy, row_stats, row_mask, s);
    default:
      return fail(ORLHF_ERR_INVALID_ARG, "logprob_entropy_bwd: unknown dtype %d", dtype);
  }
}
