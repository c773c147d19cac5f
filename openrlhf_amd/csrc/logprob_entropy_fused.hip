// Fused forward + backward of log-prob / entropy for callers that know the upstream weights
// when the forward runs (loss = sum_i w_lp[i]*logprob[i] + w_ent[i]*entropy[i]): each
// vocabulary row is read from HBM once, kept on chip, and its gradient written once, so a
// token moves 2*V*s bytes instead of the 3*V*s of a separate forward and backward.
//
// A row of 151936 bf16 logits is 297 KiB; the vector register file of one CU is 512 KiB. One
// 512-thread workgroup (8 wave64, 2 per SIMD, up to 256 VGPRs each) owns a CU and a row: every
// lane keeps 38 16-byte chunks of the row in registers (rows up to 38*512 chunks: 155648 bf16 /
// fp16 or 77824 fp32 elements). A longer row keeps its first 32*512 chunks in registers and
// streams the rest twice (once for the sums, once for the gradient, the second time from the
// caches when they still hold it): 2.5 x V bytes per token at V = 262144 instead of 3 x; rows
// beyond four times the resident part are left to the separate kernels.
#include "token_terms.h"
#include "vocab_rows.h"

namespace orlhf {

constexpr int kFusedBlock = 512;
constexpr int kFusedWaves = kFusedBlock / kWave;
constexpr int kAccF = 2;               // independent accumulators per lane
constexpr int kFusedRegChunks = 38;    // 16-byte chunks of the row each lane keeps in registers
constexpr int kFusedRegChunksLong = 32;  // the same for rows that do not fit: the rest is streamed twice
constexpr int kTailInFlight = 6;         // streamed 16-byte chunks in flight per lane (two batches of 3)
constexpr int kFusedMaxTailFactor = 4;   // longest row = 4 x the resident part; beyond, streaming three
                                         // quarters of the row twice is no better than the two kernels

constexpr int kTailHalf = kTailInFlight / 2;            // chunks per batch; two batches alternate
constexpr uint32_t kTailStep = (uint32_t)kTailHalf * 512u;  // vectors one batch covers (512 = workgroup size)

__device__ __forceinline__ u32x4 load_vec_cached(const char* p) { return *(const u32x4*)p; }

// value that contributes exp() == 0 and 0 * x == -0 (not NaN) for lanes past the row end
template <int DT>
__device__ __forceinline__ u32x4 neutral_vec() {
  if (DT == ORLHF_F32) return u32x4{0xff7fffffu, 0xff7fffffu, 0xff7fffffu, 0xff7fffffu};  // -FLT_MAX
  if (DT == ORLHF_BF16) return u32x4{0xff7fff7fu, 0xff7fff7fu, 0xff7fff7fu, 0xff7fff7fu};
  return u32x4{0xfbfffbffu, 0xfbfffbffu, 0xfbfffbffu, 0xfbfffbffu};  // fp16 -65504
}
constexpr float kNeutral = -3.0e38f;

// One batch of streamed chunks: vector v0 + u*512 + tid for u < kTailHalf, neutral past the row end.
template <int DT>
__device__ __forceinline__ void tail_load(u32x4 (&t)[kTailHalf], const char* body, uint32_t v0, uint32_t nvec,
                                          uint32_t tid) {
#pragma unroll
  for (int u = 0; u < kTailHalf; ++u) {
    const uint32_t v = v0 + (uint32_t)u * 512u + tid;
    t[u] = v < nvec ? load_vec_cached(body + v * 16u) : neutral_vec<DT>();
  }
}

// Makes the compiler forget what it knows about a resident chunk, so that every pass unpacks the
// 16-byte chunk again instead of keeping 8 fp32 values per chunk alive across passes (which
// would need three times the registers the row itself occupies). Emits no instruction.
__device__ __forceinline__ void launder(u32x4& v) {
  uint32_t a = v[0], b = v[1], c = v[2], d = v[3];
  asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
  v = u32x4{a, b, c, d};
}

// The workgroup never lets its CU's memory pipe drain: while it computes and stores the gradient
// of chunk c of row r it already issues the load of chunk c of its next row into the registers
// that chunk just left, and the sums of the next row are accumulated as those loads land. To start accumulating before the
// whole row is on chip the exponent reference is the wave maximum of each lane's first chunk (as
// in the stand-alone forward); if the sums come out non-finite the exact maximum is taken from
// the resident registers and the sums are redone, all on chip.
// Per-token loss terms of a PPO step, evaluated on the freshly computed log-prob of each row
// (TERMS kernels): the upstream weights are then d(loss)/d(logprob) and d(loss)/d(entropy) of
//   loss = sum_i policy_coef[i] * L_ppo(lp_i) + kl_coef * sum_i token_coef[i] * KL(lp_i - base_i)
//          - entropy_coef * sum_i token_coef[i] * H_i.
struct StepTerms {
  const float *old_lp, *adv, *rollout, *base, *policy_coef, *token_coef;
  PolicyTok pol;  // clip / dual-clip / importance-correction parameters (pointers unused)
  int kl_estimator;
  float kl_coef, entropy_coef;
};

template <int DT, int MODE, int REG_CHUNKS, bool TERMS, bool TAIL>
__global__ __launch_bounds__(kFusedBlock) void logprob_entropy_fused_pipe_kernel(
    const char* logits, char* grad, int64_t n_rows, int64_t vocab, int64_t row_stride_bytes,
    int64_t grad_stride_bytes, const int64_t* __restrict__ labels, double temperature,
    const float* __restrict__ w_logprob, const float* __restrict__ w_entropy,
    float* __restrict__ logprob, float* __restrict__ entropy, const uint8_t* __restrict__ row_mask,
    StepTerms terms) {
  using E = Elt<DT>;
  using MT = ModeTraits<MODE>;
  constexpr int EPV = E::kPerVec;
  constexpr uint32_t kRegVecs = (uint32_t)REG_CHUNKS * kFusedBlock;  // vectors of a row held in registers
  __shared__ float lds_max[kFusedWaves];
  __shared__ float lds_sum[kFusedWaves][8];
  __shared__ float lds_bcast[8];

  const uint32_t tid = threadIdx.x;
  const uint32_t tid16 = tid * 16u;
  const uint32_t lane = tid & (kWave - 1);
  const uint32_t wave = tid / kWave;
  const float c1 = kLog2e;
  const float cT = (float)(1.4426950408889634 / temperature);
  const double inv_t = 1.0 / temperature;

  // next row of this workgroup that is wanted; unwanted rows on the way get their zeros now
  auto next_active = [&](int64_t r) -> int64_t {
    while (r < n_rows && row_mask != nullptr && row_mask[r] == 0) {
      char* out_row = grad + r * grad_stride_bytes;
      const RowGeom gz = row_geom<DT>(logits + r * row_stride_bytes, vocab, false);
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (uint32_t v = tid; v < gz.nvec; v += kFusedBlock) store_vec(out_row + gz.head * E::kSize + v * 16u, z);
      const uint32_t nsc = gz.head + gz.tail;
      if (tid < nsc) {
        const uint32_t e = tid < gz.head ? tid : gz.head + gz.nvec * EPV + (tid - gz.head);
        E::store1(out_row + e * E::kSize, 0.0f);
      }
      if (tid == 0) {
        if (logprob != nullptr) logprob[r] = 0.0f;
        if (entropy != nullptr) entropy[r] = 0.0f;
      }
      r += gridDim.x;
    }
    return r;
  };

  u32x4 buf[REG_CHUNKS];
  float xs = kNeutral;
  int64_t row_i = next_active(blockIdx.x);
  RowGeom g = {0, 0, 0};
  if (row_i < n_rows) {  // prologue: the first row's loads
    const char* row = logits + row_i * row_stride_bytes;
    g = row_geom<DT>(row, vocab, false);
    const char* body = row + g.head * E::kSize;
#pragma unroll
    for (int c = 0; c < REG_CHUNKS; ++c) {
      const uint32_t v = (uint32_t)c * kFusedBlock + tid;
      buf[c] = v < g.nvec ? load_vec(body + (uint32_t)c * (kFusedBlock * 16u) + tid16) : neutral_vec<DT>();
    }
    const uint32_t nsc = g.head + g.tail;
    const uint32_t e = tid < g.head ? tid : g.head + g.nvec * EPV + (tid - g.head);
    xs = tid < nsc ? E::load1(row + e * E::kSize) : kNeutral;
  }

  while (row_i < n_rows) {
    const char* row = logits + row_i * row_stride_bytes;
    char* out_row = grad + row_i * grad_stride_bytes;
    char* obody = out_row + g.head * E::kSize;
    const uint32_t nscalar = g.head + g.tail;
    const uint32_t scalar_e = tid < g.head ? tid : g.head + g.nvec * EPV + (tid - g.head);

    // ---- sums against a reference; returns them combined over the workgroup
    float refT = 0.0f, ref1 = 0.0f, sumT = 0.0f, sum1 = 0.0f, sumX = 0.0f;
    auto sums = [&](float m_wave) {
      const float rT = m_wave * cT, r1 = m_wave * c1;
      const float negMT = -rT, negM1 = -r1;
      float sT[kAccF] = {0.0f, 0.0f}, s1[kAccF] = {0.0f, 0.0f}, t1[kAccF] = {0.0f, 0.0f};
      auto accumulate = [&](float x, int k) {
        if (MT::kScaledSet) sT[k] += fast_exp2(fmaf(x, cT, negMT));
        if (MT::kPlainSet) {
          const float e = fast_exp2(fmaf(x, c1, negM1));
          s1[k] += e;
          t1[k] = fmaf(e, x, t1[k]);
        }
      };
      accumulate(xs, 0);
#pragma unroll
      for (int c = 0; c < REG_CHUNKS; ++c) {
        float x[EPV];
        launder(buf[c]);
        E::unpack(buf[c], x);
#pragma unroll
        for (int j = 0; j < EPV; ++j) accumulate(x[j], j % kAccF);
      }
      if (TAIL) {  // the part of a long row that does not fit in registers is streamed (and stays cached)
        const char* tbody = row + g.head * E::kSize;
        auto consume = [&](const u32x4 (&t)[kTailHalf]) {
#pragma unroll
          for (int u = 0; u < kTailHalf; ++u) {
            float x[EPV];
            E::unpack(t[u], x);
#pragma unroll
            for (int j = 0; j < EPV; ++j) accumulate(x[j], j % kAccF);
          }
        };
        u32x4 t0[kTailHalf], t1[kTailHalf];
        uint32_t v0 = kRegVecs;
        tail_load<DT>(t0, tbody, v0, g.nvec, tid);
        while (v0 < g.nvec) {  // two batches alternate: one is in flight while the other is consumed
          tail_load<DT>(t1, tbody, v0 + kTailStep, g.nvec, tid);
          consume(t0);
          v0 += kTailStep;
          if (v0 >= g.nvec) break;
          tail_load<DT>(t0, tbody, v0 + kTailStep, g.nvec, tid);
          consume(t1);
          v0 += kTailStep;
        }
      }
      const float wst = wave_sum(sT[0] + sT[1]);
      const float ws1 = wave_sum(s1[0] + s1[1]);
      const float wt1 = wave_sum(t1[0] + t1[1]);
      if (lane == 0) {
        lds_sum[wave][0] = rT;
        lds_sum[wave][1] = wst;
        lds_sum[wave][2] = r1;
        lds_sum[wave][3] = ws1;
        lds_sum[wave][4] = wt1;
      }
      __syncthreads();
      float MTm = lds_sum[0][0], M1m = lds_sum[0][2];
#pragma unroll
      for (int w = 1; w < kFusedWaves; ++w) {
        MTm = fmaxf(MTm, lds_sum[w][0]);
        M1m = fmaxf(M1m, lds_sum[w][2]);
      }
      sumT = sum1 = sumX = 0.0f;
#pragma unroll
      for (int w = 0; w < kFusedWaves; ++w) {
        const float qT = fast_exp2(lds_sum[w][0] - MTm);
        const float q1 = fast_exp2(lds_sum[w][2] - M1m);
        sumT = fmaf(lds_sum[w][1], qT, sumT);
        sum1 = fmaf(lds_sum[w][3], q1, sum1);
        sumX = fmaf(lds_sum[w][4], q1, sumX);
      }
      refT = MTm;
      ref1 = M1m;
      __syncthreads();
    };

    // reference = wave maximum of each lane's first chunk (lands first), exact maximum if needed
    {
      float x[EPV];
      E::unpack(buf[0], x);
      float m0 = x[0];
#pragma unroll
      for (int j = 1; j < EPV; ++j) m0 = fmaxf(m0, x[j]);
      sums(wave_max(fmaxf(m0, xs)));
    }
    bool ok = true;
    if (MT::kScaledSet) ok = ok && (sumT > 0.0f && sumT < INFINITY);
    if (MT::kPlainSet) ok = ok && (sum1 > 0.0f && sum1 < INFINITY) && (fabsf(sumX) < INFINITY);
    bool plus_inf_row = false;  // maximum +inf and no NaN: logsumexp is +inf, softmax undefined
    if (!ok) {  // workgroup-uniform, rare: the row is on chip, take its exact maximum
      float m = xs;
      bool nan_seen = xs != xs;
#pragma unroll
      for (int c = 0; c < REG_CHUNKS; ++c) {
        float x[EPV];
        launder(buf[c]);
        E::unpack(buf[c], x);
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
          m = fmaxf(m, x[j]);
          nan_seen = nan_seen || (x[j] != x[j]);
        }
      }
      if (TAIL) {
        const char* tbody = row + g.head * E::kSize;
        for (uint32_t v = kRegVecs + tid; v < g.nvec; v += kFusedBlock) {
          float x[EPV];
          E::unpack(load_vec_cached(tbody + v * 16u), x);
#pragma unroll
          for (int j = 0; j < EPV; ++j) {
            m = fmaxf(m, x[j]);
            nan_seen = nan_seen || (x[j] != x[j]);
          }
        }
      }
      m = wave_max(m);
      const bool wave_nan = __ballot(nan_seen) != 0ull;
      if (lane == 0) {
        lds_max[wave] = m;
        lds_sum[wave][5] = wave_nan ? 1.0f : 0.0f;
      }
      __syncthreads();
      m = lds_max[0];
      float nans = lds_sum[0][5];
#pragma unroll
      for (int w = 1; w < kFusedWaves; ++w) {
        m = fmaxf(m, lds_max[w]);
        nans += lds_sum[w][5];
      }
      plus_inf_row = (m == INFINITY) && (nans == 0.0f);
      sums(m);
    }

    // ---- row statistics, outputs and gradient coefficients (one lane, fp64), broadcast
    if (tid == 0) {
      double lse_t = 0.0, lse_1 = 0.0, ex = 0.0;
      if (MT::kScaledSet) lse_t = (double)refT * kLn2d + log((double)sumT);
      if (MT::kPlainSet) {
        lse_1 = (double)ref1 * kLn2d + log((double)sum1);
        ex = (double)sumX / (double)sum1;
        if (!MT::kScaledSet) lse_t = lse_1;
      }
      if (plus_inf_row) {  // what torch.logsumexp / softmax give for a +inf logit
        lse_t = lse_1 = INFINITY;
        ex = NAN;
      }
      const int64_t label = (MODE != kEntOnly) ? labels[row_i] : -1;
      float lp = 0.0f;
      if (MODE != kEntOnly) {
        if (label >= 0 && label < vocab)
          lp = (float)((double)E::load1(row + label * E::kSize) * inv_t - lse_t);
        else
          lp = (label == -100) ? 0.0f : NAN;
        if (logprob != nullptr) logprob[row_i] = lp;
      }
      if (MT::kPlainSet && entropy != nullptr) entropy[row_i] = (float)(lse_1 - ex);
      float glp = 0.0f, gh = 0.0f;
      if (TERMS) {
        const float pc = terms.policy_coef[row_i];
        const float tc = terms.token_coef[row_i];
        if (pc != 0.0f) {
          const float old_v = terms.old_lp[row_i];
          const float w = terms.rollout != nullptr ? terms.pol.token_is_weight_of(old_v, terms.rollout[row_i]) : 1.0f;
          glp = pc * terms.pol.ppo_grad_of(lp, old_v, terms.adv[row_i], w);
        }
        if (tc != 0.0f) {
          if (terms.base != nullptr) {
            float kv, kd;
            kl_value(terms.kl_estimator, lp - terms.base[row_i], kv, kd);
            glp += terms.kl_coef * tc * kd;
          }
          gh = -terms.entropy_coef * tc;
        }
      } else {
        glp = (MODE != kEntOnly && w_logprob != nullptr) ? w_logprob[row_i] : 0.0f;
        gh = (MT::kPlainSet && w_entropy != nullptr) ? w_entropy[row_i] : 0.0f;
      }
      lds_bcast[0] = -(float)(lse_t * 1.4426950408889634);
      lds_bcast[1] = -(float)(lse_1 * 1.4426950408889634);
      lds_bcast[2] = -(float)((double)glp * inv_t);
      lds_bcast[3] = (float)((double)glp * inv_t);
      lds_bcast[4] = gh;
      lds_bcast[5] = gh * (float)ex - (MODE == kBothT1 ? glp : 0.0f);
    }
    __syncthreads();
    GradFn<MODE> fn;
    fn.cT = cT;
    fn.c1 = c1;
    fn.negLT = lds_bcast[0];
    fn.negL1 = lds_bcast[1];
    fn.a_lp = lds_bcast[2];
    fn.onehot = lds_bcast[3];
    fn.gh = lds_bcast[4];
    fn.k1 = lds_bcast[5];
    fn.set_label((MODE != kEntOnly) ? labels[row_i] : -1, vocab, g, EPV);

    // ---- gradient of this row out, next row in, chunk by chunk through the same registers
    const int64_t next_i = next_active(row_i + gridDim.x);
    const bool has_next = next_i < n_rows;
    const char* nrow = logits + (has_next ? next_i : row_i) * row_stride_bytes;
    const RowGeom gn = has_next ? row_geom<DT>(nrow, vocab, false) : RowGeom{0, 0, 0};
    const char* nbody = nrow + gn.head * E::kSize;
#pragma unroll
    for (int c = 0; c < REG_CHUNKS; ++c) {
      const uint32_t v = (uint32_t)c * kFusedBlock + tid;
      if (v < g.nvec) {
        float x[EPV];
        launder(buf[c]);
        E::unpack(buf[c], x);
        fn.vec(x, v);
        store_vec(obody + (uint32_t)c * (kFusedBlock * 16u) + tid16, E::pack(x));
      }
      buf[c] = v < gn.nvec ? load_vec(nbody + (uint32_t)c * (kFusedBlock * 16u) + tid16) : neutral_vec<DT>();
    }
    if (TAIL) {  // the streamed part again (from the caches when they still hold it), then its gradient
      const char* tbody = row + g.head * E::kSize;
      auto emit = [&](const u32x4 (&t)[kTailHalf], uint32_t base) {
#pragma unroll
        for (int u = 0; u < kTailHalf; ++u) {
          const uint32_t v = base + (uint32_t)u * kFusedBlock + tid;
          if (v < g.nvec) {
            float x[EPV];
            E::unpack(t[u], x);
            fn.vec(x, v);
            store_vec(obody + v * 16u, E::pack(x));
          }
        }
      };
      u32x4 t0[kTailHalf], t1[kTailHalf];
      uint32_t v0 = kRegVecs;
      tail_load<DT>(t0, tbody, v0, g.nvec, tid);
      while (v0 < g.nvec) {
        tail_load<DT>(t1, tbody, v0 + kTailStep, g.nvec, tid);
        emit(t0, v0);
        v0 += kTailStep;
        if (v0 >= g.nvec) break;
        tail_load<DT>(t0, tbody, v0 + kTailStep, g.nvec, tid);
        emit(t1, v0);
        v0 += kTailStep;
      }
    }
    if (tid < nscalar) {
      fn.one(xs, scalar_e);
      E::store1(out_row + scalar_e * E::kSize, xs);
    }
    {
      const uint32_t nsc = gn.head + gn.tail;
      const uint32_t e = tid < gn.head ? tid : gn.head + gn.nvec * EPV + (tid - gn.head);
      xs = tid < nsc ? E::load1(nrow + e * E::kSize) : kNeutral;
    }
    row_i = next_i;
    g = gn;
  }
}

template <int DT>
static int launch_fused(const void* logits, void* grad, int64_t n_rows, int64_t vocab, int64_t row_stride,
                        int64_t grad_row_stride, const int64_t* labels, double temperature,
                        const float* w_logprob, const float* w_entropy, float* logprob, float* entropy,
                        const uint8_t* row_mask, const StepTerms* terms, int n_cu, hipStream_t stream) {
  using E = Elt<DT>;
  const bool want_ent = entropy != nullptr || w_entropy != nullptr || (terms != nullptr && terms->entropy_coef != 0.0f);
  const bool want_lp = logprob != nullptr || w_logprob != nullptr || terms != nullptr;
  const bool t1 = (temperature == 1.0);
  const int mode = !want_ent ? kLpOnly : (!want_lp ? kEntOnly : (t1 ? kBothT1 : kBothT));
  const char* p = (const char*)logits;
  char* gp = (char*)grad;
  const int64_t sb = row_stride * E::kSize, gsb = grad_row_stride * E::kSize;
  // one workgroup per CU (it takes the whole register file), walking rows grid-stride
  const int64_t blocks = n_rows < n_cu ? n_rows : n_cu;
  const dim3 grid((unsigned)blocks), block(kFusedBlock);
  StepTerms none = {};
  const bool long_rows = vocab > (int64_t)kFusedRegChunks * kFusedBlock * E::kPerVec;
#define ORLHF_FUSED_ARGS                                                                                        \
  grid, block, 0, stream, p, gp, n_rows, vocab, sb, gsb, labels, temperature, w_logprob, w_entropy, logprob, entropy, \
      row_mask
#define ORLHF_FUSED(M)                                                                                             \
  if (long_rows && terms != nullptr)                                                                               \
    hipLaunchKernelGGL((logprob_entropy_fused_pipe_kernel<DT, M, kFusedRegChunksLong, true, true>), ORLHF_FUSED_ARGS, *terms); \
  else if (long_rows)                                                                                              \
    hipLaunchKernelGGL((logprob_entropy_fused_pipe_kernel<DT, M, kFusedRegChunksLong, false, true>), ORLHF_FUSED_ARGS, none); \
  else if (terms != nullptr)                                                                                       \
    hipLaunchKernelGGL((logprob_entropy_fused_pipe_kernel<DT, M, kFusedRegChunks, true, false>), ORLHF_FUSED_ARGS, *terms); \
  else                                                                                                             \
    hipLaunchKernelGGL((logprob_entropy_fused_pipe_kernel<DT, M, kFusedRegChunks, false, false>), ORLHF_FUSED_ARGS, none)
  switch (mode) {
    case kLpOnly: ORLHF_FUSED(kLpOnly); break;
    case kEntOnly: ORLHF_FUSED(kEntOnly); break;
    case kBothT1: ORLHF_FUSED(kBothT1); break;
    default: ORLHF_FUSED(kBothT); break;
  }
#undef ORLHF_FUSED
#undef ORLHF_FUSED_ARGS
  ORLHF_CHECK_LAUNCH("orlhf_logprob_entropy_fwd_bwd");
  return ORLHF_OK;
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int64_t orlhf_logprob_entropy_fwd_bwd_max_vocab(int dtype) {
  const int64_t per_vec = dtype == ORLHF_F32 ? 4 : 8;
  if (dtype != ORLHF_F32 && dtype != ORLHF_BF16 && dtype != ORLHF_F16) return 0;
  return (int64_t)kFusedMaxTailFactor * kFusedRegChunksLong * kFusedBlock * per_vec;
}

static int fused_entry(const void* logits, void* grad_logits, int dtype, int64_t n_rows, int64_t vocab,
                       int64_t row_stride, int64_t grad_row_stride, const int64_t* labels, double temperature,
                       const float* w_logprob, const float* w_entropy, float* logprob, float* entropy,
                       const uint8_t* row_mask, const StepTerms* terms, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && vocab > 0, "logprob_entropy_fwd_bwd: n_rows=%lld vocab=%lld", (long long)n_rows,
                  (long long)vocab);
  ORLHF_CHECK_ARG(row_stride >= vocab && grad_row_stride >= vocab,
                  "logprob_entropy_fwd_bwd: row strides %lld/%lld < vocab %lld", (long long)row_stride,
                  (long long)grad_row_stride, (long long)vocab);
  ORLHF_CHECK_ARG(temperature > 0.0 && temperature == temperature, "logprob_entropy_fwd_bwd: temperature must be > 0");
  ORLHF_CHECK_ARG(dtype == ORLHF_F32 || dtype == ORLHF_BF16 || dtype == ORLHF_F16,
                  "logprob_entropy_fwd_bwd: unknown dtype %d", dtype);
  if (n_rows == 0) return ORLHF_OK;  // nothing to launch; empty arrays may well be NULL
  ORLHF_CHECK_ARG(terms != nullptr || w_logprob != nullptr || w_entropy != nullptr || logprob != nullptr ||
                      entropy != nullptr,
                  "logprob_entropy_fwd_bwd: nothing to compute");
  ORLHF_CHECK_ARG(logits != nullptr && grad_logits != nullptr, "logprob_entropy_fwd_bwd: NULL logits / grad_logits");
  ORLHF_CHECK_ARG((logprob == nullptr && w_logprob == nullptr && terms == nullptr) || labels != nullptr,
                  "logprob_entropy_fwd_bwd: labels is NULL");
  const int esize = dtype == ORLHF_F32 ? 4 : 2;
  ORLHF_CHECK_ARG((((uintptr_t)logits | (uintptr_t)grad_logits) & (uintptr_t)(esize - 1)) == 0,
                  "logprob_entropy_fwd_bwd: pointers not aligned to the element size");
  if (vocab > orlhf_logprob_entropy_fwd_bwd_max_vocab(dtype))
    return fail(ORLHF_ERR_UNSUPPORTED,
                "logprob_entropy_fwd_bwd: a row of %lld elements is too long for the one-pass kernel (max %lld); "
                "use the separate forward and backward",
                (long long)vocab, (long long)orlhf_logprob_entropy_fwd_bwd_max_vocab(dtype));
  const bool same_phase = (((uintptr_t)logits ^ (uintptr_t)grad_logits) & 15u) == 0 &&
                          (((row_stride - grad_row_stride) * esize) & 15) == 0;
  if (!same_phase)
    return fail(ORLHF_ERR_UNSUPPORTED,
                "logprob_entropy_fwd_bwd: logits and grad rows sit on different 16-byte phases; use the separate "
                "forward and backward");
  int device = 0, n_cu = 256;
  if (hipGetDevice(&device) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) n_cu = v;
  }
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case ORLHF_F32:
      return launch_fused<ORLHF_F32>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride, labels,
                                     temperature, w_logprob, w_entropy, logprob, entropy, row_mask, terms, n_cu, s);
    case ORLHF_BF16:
      return launch_fused<ORLHF_BF16>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride, labels,
                                      temperature, w_logprob, w_entropy, logprob, entropy, row_mask, terms, n_cu, s);
    default:
      return launch_fused<ORLHF_F16>(logits, grad_logits, n_rows, vocab, row_stride, grad_row_stride, labels,
                                     temperature, w_logprob, w_entropy, logprob, entropy, row_mask, terms, n_cu, s);
  }
}


extern "C" int orlhf_logprob_entropy_fwd_bwd(const void* logits, void* grad_logits, int dtype, int64_t n_rows,
                                             int64_t vocab, int64_t row_stride, int64_t grad_row_stride,
                                             const int64_t* labels, double temperature, const float* w_logprob,
                                             const float* w_entropy, float* logprob, float* entropy,
                                             const uint8_t* row_mask, orlhf_stream_t stream) {
  return fused_entry(logits, grad_logits, dtype, n_rows, vocab, row_stride, grad_row_stride, labels, temperature,
                     w_logprob, w_entropy, logprob, entropy, row_mask, nullptr, stream);
}

extern "C" int orlhf_policy_step_fwd_bwd(const void* logits, void* grad_logits, int dtype, int64_t n_rows,
                                         int64_t vocab, int64_t row_stride, int64_t grad_row_stride,
                                         const int64_t* labels, double temperature, const orlhf_step_terms* t,
                                         float* logprob, float* entropy, const uint8_t* row_mask,
                                         orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(t != nullptr, "policy_step_fwd_bwd: terms is NULL");
  ORLHF_CHECK_ARG(n_rows == 0 || (t->old_log_probs && t->advantages && t->policy_coef && t->token_coef),
                  "policy_step_fwd_bwd: old_log_probs / advantages / policy_coef / token_coef must be given");
  ORLHF_CHECK_ARG(t->is_correction == ORLHF_IS_NONE || t->is_correction == ORLHF_IS_TIS ||
                      t->is_correction == ORLHF_IS_ICEPOP,
                  "policy_step_fwd_bwd: only token-level importance corrections (none, tis, icepop) can be fused, got %d",
                  t->is_correction);
  ORLHF_CHECK_ARG(t->is_correction == ORLHF_IS_NONE || t->rollout_log_probs != nullptr,
                  "policy_step_fwd_bwd: importance correction needs rollout_log_probs");
  ORLHF_CHECK_ARG(t->base_log_probs == nullptr || (t->kl_estimator >= ORLHF_KL_K1 && t->kl_estimator <= ORLHF_KL_K3),
                  "policy_step_fwd_bwd: unknown kl_estimator %d", t->kl_estimator);
  ORLHF_CHECK_ARG(!(t->dual_clip > 0.0f) || t->dual_clip > 1.0f, "policy_step_fwd_bwd: dual_clip must be > 1.0, got %g",
                  (double)t->dual_clip);
  StepTerms st = {};
  st.old_lp = t->old_log_probs;
  st.adv = t->advantages;
  st.rollout = t->is_correction == ORLHF_IS_NONE ? nullptr : t->rollout_log_probs;
  st.base = t->base_log_probs;
  st.policy_coef = t->policy_coef;
  st.token_coef = t->token_coef;
  st.pol.lp = st.pol.old = st.pol.adv = st.pol.rollout = st.pol.row_aux = nullptr;
  st.pol.lo = 1.0f - t->clip_eps_low;
  st.pol.hi = 1.0f + t->clip_eps_high;
  st.pol.dual = t->dual_clip;
  st.pol.gspo = 0;
  st.pol.is_mode = t->is_correction;
  st.pol.is_lo = t->is_low;
  st.pol.is_hi = t->is_high;
  st.kl_estimator = t->kl_estimator;
  st.kl_coef = t->kl_coef;
  st.entropy_coef = t->entropy_coef;
  return fused_entry(logits, grad_logits, dtype, n_rows, vocab, row_stride, grad_row_stride, labels, temperature,
                     nullptr, nullptr, logprob, entropy, row_mask, &st, stream);
}

// ---------------------------------------------------------------- conditional in-place rescale
namespace orlhf {
template <int DT>
__global__ __launch_bounds__(kBlock) void rescale_if_kernel(char* data, int64_t n, const float* __restrict__ g,
                                                            float expected) {
  using E = Elt<DT>;
  const float f = g[0] / expected;
  if (f == 1.0f) return;  // the usual case: the gradient was produced with the right scale
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    E::store1(data + i * E::kSize, E::load1(data + i * E::kSize) * f);
}
}  // namespace orlhf

extern "C" int orlhf_rescale_inplace_if(void* data, int dtype, int64_t n, const float* g, float expected,
                                        orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0 && expected != 0.0f && expected == expected, "rescale_inplace_if: n=%lld expected=%g",
                  (long long)n, (double)expected);
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(data != nullptr && g != nullptr, "rescale_inplace_if: NULL pointer");
  const dim3 grid(flat_grid(n, 16384)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case ORLHF_F32: hipLaunchKernelGGL(rescale_if_kernel<ORLHF_F32>, grid, block, 0, s, (char*)data, n, g, expected); break;
    case ORLHF_BF16: hipLaunchKernelGGL(rescale_if_kernel<ORLHF_BF16>, grid, block, 0, s, (char*)data, n, g, expected); break;
    case ORLHF_F16: hipLaunchKernelGGL(rescale_if_kernel<ORLHF_F16>, grid, block, 0, s, (char*)data, n, g, expected); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "rescale_inplace_if: unknown dtype %d", dtype);
  }
  ORLHF_CHECK_LAUNCH("orlhf_rescale_inplace_if");
  return ORLHF_OK;
}
