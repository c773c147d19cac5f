// Shared pieces of the vocabulary-row kernels: element traits (bf16 / fp16 / fp32 as 16-byte
// vectors), row geometry, statistic modes and the per-element gradient.
#pragma once
#include "common.h"

#ifndef ORLHF_NT_LOAD
#define ORLHF_NT_LOAD 1
#endif
#ifndef ORLHF_NT_STORE
#define ORLHF_NT_STORE 1
#endif

namespace orlhf {

// ---------------------------------------------------------------- element traits
template <int DT>
struct Elt;

template <>
struct Elt<ORLHF_BF16> {
  static constexpr int kSize = 2;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float (&x)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x[2 * k] = bf16_lo(r[k]);
      x[2 * k + 1] = bf16_hi(r[k]);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&x)[8]) {
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = pack_bf16(x[2 * k], x[2 * k + 1]);
    return r;
  }
  static __device__ __forceinline__ float load1(const char* p) {
    return __builtin_bit_cast(float, (uint32_t)(*(const uint16_t*)p) << 16);
  }
  static __device__ __forceinline__ void store1(char* p, float v) {
    *(uint16_t*)p = (uint16_t)(pack_bf16(v, 0.0f) & 0xffffu);
  }
  static __device__ __forceinline__ float round(float v) { return bf16_lo(pack_bf16(v, 0.0f)); }
};

template <>
struct Elt<ORLHF_F16> {
  static constexpr int kSize = 2;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float (&x)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t w = r[k];  // by value: a vector lane is not addressable
      f16x2 h = __builtin_bit_cast(f16x2, w);
      x[2 * k] = (float)h[0];
      x[2 * k + 1] = (float)h[1];
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&x)[8]) {
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = pack_f16(x[2 * k], x[2 * k + 1]);
    return r;
  }
  static __device__ __forceinline__ float load1(const char* p) { return (float)(*(const _Float16*)p); }
  static __device__ __forceinline__ void store1(char* p, float v) { *(_Float16*)p = (_Float16)v; }
  static __device__ __forceinline__ float round(float v) { return (float)(_Float16)v; }
};

template <>
struct Elt<ORLHF_F32> {
  static constexpr int kSize = 4;
  static constexpr int kPerVec = 4;
  static __device__ __forceinline__ void unpack(const u32x4& r, float (&x)[4]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) x[k] = as_float(r[k]);  // by value: a vector lane is not addressable
  }
  static __device__ __forceinline__ u32x4 pack(const float (&x)[4]) {
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = as_uint(x[k]);
    return r;
  }
  static __device__ __forceinline__ float load1(const char* p) { return *(const float*)p; }
  static __device__ __forceinline__ void store1(char* p, float v) { *(float*)p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

__device__ __forceinline__ u32x4 load_vec(const char* p) {
#if ORLHF_NT_LOAD
  return __builtin_nontemporal_load((const u32x4*)p);
#else
  return *(const u32x4*)p;
#endif
}
__device__ __forceinline__ void store_vec(char* p, const u32x4& v) {
#if ORLHF_NT_STORE
  __builtin_nontemporal_store(v, (u32x4*)p);
#else
  *(u32x4*)p = v;
#endif
}

// ---------------------------------------------------------------- row geometry + traversal
// A row is split into a scalar head (elements before the first 16-byte boundary), a body of
// 16-byte vectors and a scalar tail, so any vocab size, row stride and base alignment works.
// `scalar_only` (host decision: input and output rows are misaligned differently) turns the
// whole row into the scalar part.
struct RowGeom {
  uint32_t head, nvec, tail;  // element / vector counts; a row is < 2 GiB (host check)
};

template <int DT>
__device__ __forceinline__ RowGeom row_geom(const char* row, int64_t vocab, bool scalar_only) {
  using E = Elt<DT>;
  RowGeom g;
  if (scalar_only) {
    g.head = (uint32_t)vocab;
    g.nvec = 0;
    g.tail = 0;
    return g;
  }
  const uint32_t mis = (uint32_t)((uintptr_t)row & 15u);
  uint32_t head = mis ? (16u - mis) / E::kSize : 0u;
  if (head > (uint32_t)vocab) head = (uint32_t)vocab;
  g.head = head;
  g.nvec = ((uint32_t)vocab - head) / E::kPerVec;
  g.tail = (uint32_t)vocab - head - g.nvec * E::kPerVec;
  return g;
}

// ---------------------------------------------------------------- forward accumulators
// Modes: which statistics a row needs.
//   kLpOnly   : sum exp(z - m)                      z = x / T
//   kEntOnly  : sum exp(x - m), sum exp(x - m) * x
//   kBothT1   : T == 1, one shared set
//   kBothT    : T != 1, scaled set for the log-prob and unscaled set for the entropy
enum FwdMode { kLpOnly = 0, kEntOnly = 1, kBothT1 = 2, kBothT = 3 };

template <int MODE>
struct ModeTraits {
  static constexpr bool kScaledSet = (MODE == kLpOnly || MODE == kBothT);  // separate x/T set
  static constexpr bool kPlainSet = (MODE != kLpOnly);                     // unscaled set (+ sum e*x)
};

// ---------------------------------------------------------------- gradient of one element
enum BwdMode { kBwdLp = 0, kBwdEnt = 1, kBwdBothT1 = 2, kBwdBothT = 3 };

template <int MODE>
struct GradFn {
  float cT, negLT, c1, negL1;  // exponents: x*c - lse*log2e
  float a_lp;                  // -g_lp / T          (coefficient of softmax(z))
  float gh, k1;                // entropy term p*(k1 - gh*x); k1 = gh*E (- g_lp when T == 1)
  float onehot;                // g_lp / T
  uint32_t label_vec;          // body vector holding the label (0xffffffff: none)
  uint32_t label_lane;         // its position inside that vector
  uint32_t label_elem;         // the label as an element index (0xffffffff: out of range)
  __device__ __forceinline__ float elem(float x) const {
    if (MODE == kBwdLp) return fast_exp2(fmaf(x, cT, negLT)) * a_lp;
    if (MODE == kBwdEnt || MODE == kBwdBothT1) return fast_exp2(fmaf(x, c1, negL1)) * fmaf(-gh, x, k1);
    const float pt = fast_exp2(fmaf(x, cT, negLT));
    const float p1 = fast_exp2(fmaf(x, c1, negL1));
    return fmaf(pt, a_lp, p1 * fmaf(-gh, x, k1));
  }
  template <int N>
  __device__ __forceinline__ void vec(float (&x)[N], uint32_t v) const {
#pragma unroll
    for (int j = 0; j < N; ++j) x[j] = elem(x[j]);
    if (MODE != kBwdEnt && v == label_vec) {
#pragma unroll
      for (int j = 0; j < N; ++j) x[j] += ((uint32_t)j == label_lane) ? onehot : 0.0f;
    }
  }
  __device__ __forceinline__ void one(float& x, uint32_t e) const {
    x = elem(x);
    if (MODE != kBwdEnt && e == label_elem) x += onehot;
  }
  __device__ __forceinline__ void set_label(int64_t label, int64_t vocab, const RowGeom& g, int epv) {
    label_vec = label_lane = label_elem = 0xffffffffu;
    if (label < 0 || label >= vocab) return;
    label_elem = (uint32_t)label;
    if (label_elem >= g.head && label_elem < g.head + g.nvec * (uint32_t)epv) {
      label_vec = (label_elem - g.head) / (uint32_t)epv;
      label_lane = (label_elem - g.head) % (uint32_t)epv;
    }
  }
};

}  // namespace orlhf
