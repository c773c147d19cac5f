// Shared device/host helpers for the gfx950 (CDNA4, wave64) token-numerics kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/openrlhf_amd.h"

namespace orlhf {

constexpr int kWave = 64;       // CDNA wavefront width
constexpr int kBlock = 256;     // 4 wave64 per workgroup: one wave per SIMD of a CU
constexpr int kWavesPerBlock = kBlock / kWave;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr double kLn2d = 0.6931471805599453;

// ---------------------------------------------------------------- error state
// Thread-local message behind orlhf_last_error(); set by every failing entry point.
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define ORLHF_CHECK_ARG(cond, ...)                              \
  do {                                                          \
    if (!(cond)) return ::orlhf::fail(ORLHF_ERR_INVALID_ARG, __VA_ARGS__); \
  } while (0)

#define ORLHF_CHECK_LAUNCH(name)                                                     \
  do {                                                                               \
    hipError_t e_ = hipGetLastError();                                               \
    if (e_ != hipSuccess)                                                            \
      return ::orlhf::fail(ORLHF_ERR_LAUNCH, "%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

// ---------------------------------------------------------------- wave / block reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a whole kBlock-thread workgroup; every thread gets the result. `lds` holds
// kWavesPerBlock doubles and may be reused after the call returns (trailing barrier).
__device__ __forceinline__ double block_sum(double v, double* lds) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  double r = 0.0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) r += lds[w];
  __syncthreads();
  return r;
}

// ---------------------------------------------------------------- dtype helpers
__device__ __forceinline__ float as_float(uint32_t w) { return __builtin_bit_cast(float, w); }
__device__ __forceinline__ uint32_t as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// Two fp32 -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

// Raw v_exp_f32 (2^x); inputs below -126 flush to zero, which is what the callers want.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Mask element as a float weight; the reference multiplies by the mask, so a float mask
// acts as a weight and a bool mask as 0/1.
template <int MASK_DT>
__device__ __forceinline__ float load_mask(const void* mask, int64_t i) {
  if (MASK_DT == ORLHF_MASK_NONE) return 1.0f;
  if (MASK_DT == ORLHF_MASK_U8) return (float)((const uint8_t*)mask)[i];
  if (MASK_DT == ORLHF_MASK_F32) return ((const float*)mask)[i];
  return (float)((const int64_t*)mask)[i];
}

inline bool valid_mask_dtype(int m) { return m >= ORLHF_MASK_NONE && m <= ORLHF_MASK_I64; }

// Expands LAUNCH(M) with M = the compile-time mask dtype matching `mask_dt` (validated before by
// check_rows); LAUNCH is a function-like macro the caller defines around its kernel launch.
#define ORLHF_FOR_MASK_DTYPE(mask_dt, LAUNCH)              \
  switch (mask_dt) {                                       \
    case ORLHF_MASK_NONE: LAUNCH(ORLHF_MASK_NONE); break;  \
    case ORLHF_MASK_U8: LAUNCH(ORLHF_MASK_U8); break;      \
    case ORLHF_MASK_F32: LAUNCH(ORLHF_MASK_F32); break;    \
    default: LAUNCH(ORLHF_MASK_I64); break;                \
  }

// ---------------------------------------------------------------- per-token row layouts
// padded: contiguous [n_rows, n_cols]; packed: row b = tokens cu[b] .. cu[b+1]-1 of a flat array.
struct Rows {
  int64_t n_rows, n_cols;
  const int64_t* cu;  // packed layout when non-null
  int chunk = 0;      // chunked kernels: tokens of one row per work item
  const int64_t* order = nullptr;  // one-workgroup-per-row kernels: slot s works on row order[s] (a permutation)
};

__device__ __forceinline__ void row_span(const Rows& r, int64_t b, int64_t& start, int64_t& len) {
  if (r.cu != nullptr) {
    start = r.cu[b];
    len = r.cu[b + 1] - start;
  } else {
    start = b * r.n_cols;
    len = r.n_cols;
  }
}

// ---------------------------------------------------------------- four tokens per lane
// Kernels whose lanes work on four consecutive tokens load them with one 16-byte instruction per
// fp32 array and one load of the four mask elements. The vector types below promise only the
// element's own alignment: gfx950 global memory takes such accesses as one instruction wherever
// they start, so rows that begin anywhere (packed layouts) and arrays at any address take the
// same path. Walking every row from the 16-byte boundary before it instead was measured slower
// (one more step per row; the scans 10-15 % on ragged packed batches).
typedef float f32x4e __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2h __attribute__((ext_vector_type(2), aligned(2)));  // four 2-byte elements
typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
typedef int64_t i64x2e __attribute__((ext_vector_type(2), aligned(8)));
typedef uint32_t u32_b __attribute__((aligned(1)));  // four 1-byte elements

// Four consecutive floats that this kernel reads once: a non-temporal load, so that the stream
// does not push out of the caches what is read again (PolicyLoss forward 150 -> 131 us on 67 M
// tokens). Arrays that a later pass of the same kernel re-reads are loaded the plain way.
__device__ __forceinline__ f32x4 stream_load4(const float* p) {
  return __builtin_nontemporal_load((const f32x4e*)p);
}

// STREAM = false: cached loads, for a lane that comes back to the same cache lines with its next
// load (two groups of four tokens per lane): non-temporal there fetches the lines twice.
// One overload per element-aligned type: the parameter keeps the typedef, so the load inside is
// compiled with the element's alignment, not the natural alignment of the vector.
template <bool STREAM>
__device__ __forceinline__ f32x4 load_once(const f32x4e* p) {
  return STREAM ? __builtin_nontemporal_load(p) : *p;
}
template <bool STREAM>
__device__ __forceinline__ i64x2 load_once(const i64x2e* p) {
  return STREAM ? __builtin_nontemporal_load(p) : *p;
}
template <bool STREAM>
__device__ __forceinline__ uint32_t load_once(const u32_b* p) {
  return STREAM ? __builtin_nontemporal_load(p) : *p;
}

template <int MASK_DT, bool STREAM = true>
__device__ __forceinline__ void load_mask4(const void* mask, int64_t i0, float* m) {
  if (MASK_DT == ORLHF_MASK_NONE) {
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = 1.0f;
  } else if (MASK_DT == ORLHF_MASK_U8) {
    const uint32_t w = load_once<STREAM>((const u32_b*)((const uint8_t*)mask + i0));
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = (float)((w >> (8 * k)) & 0xffu);
  } else if (MASK_DT == ORLHF_MASK_F32) {
    const f32x4 x = load_once<STREAM>((const f32x4e*)((const float*)mask + i0));
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = x[k];
  } else {
    const i64x2 lo = load_once<STREAM>((const i64x2e*)((const int64_t*)mask + i0)),
                hi = load_once<STREAM>((const i64x2e*)((const int64_t*)mask + i0 + 2));
    m[0] = (float)lo[0];
    m[1] = (float)lo[1];
    m[2] = (float)hi[0];
    m[3] = (float)hi[1];
  }
}

// A row as the kernels walk it: flat index of its first token and its length.
struct RowWalk {
  int64_t base, len;
};
__device__ __forceinline__ RowWalk row_walk(const Rows& rows, int64_t b) {
  RowWalk w;
  row_span(rows, b, w.base, w.len);
  if (w.len < 0) w.len = 0;
  return w;
}

// A log-prob element of dtype DT (ORLHF_F32 / ORLHF_BF16 / ORLHF_F16) as fp32.
template <int DT>
__device__ __forceinline__ float load_lp(const void* p, int64_t i) {
  if (DT == ORLHF_F32) return ((const float*)p)[i];
  if (DT == ORLHF_BF16) return as_float((uint32_t)((const uint16_t*)p)[i] << 16);
  return (float)((const _Float16*)p)[i];
}

// four consecutive elements from index i0
template <int DT>
__device__ __forceinline__ void load_lp4(const void* p, int64_t i0, float* v) {
  if (DT == ORLHF_F32) {
    const f32x4 x = stream_load4((const float*)p + i0);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = x[k];
  } else {
    const u32x2 w = __builtin_nontemporal_load((const u32x2h*)((const uint16_t*)p + i0));
    if (DT == ORLHF_BF16) {
      v[0] = bf16_lo(w[0]), v[1] = bf16_hi(w[0]), v[2] = bf16_lo(w[1]), v[3] = bf16_hi(w[1]);
    } else {
      const f16x2 a = __builtin_bit_cast(f16x2, w[0]), b = __builtin_bit_cast(f16x2, w[1]);
      v[0] = (float)a[0], v[1] = (float)a[1], v[2] = (float)b[0], v[3] = (float)b[1];
    }
  }
}

// Walks one row with the whole workgroup, four consecutive tokens per lane and step: four(i0)
// where all four lie in the row (flat index i0 of the first), one(i) for the tokens of the lane
// that meets the row's end. Every token of the row is visited exactly once.
template <typename F4, typename F1>
__device__ __forceinline__ void for_row_tokens(const RowWalk& rw, F4&& four, F1&& one) {
  constexpr int kStep = kBlock * 4;
  int64_t s0 = 0;
#pragma unroll 2
  for (; s0 + kStep <= rw.len; s0 += kStep) four(rw.base + s0 + (int64_t)threadIdx.x * 4);
  if (s0 < rw.len) {  // the last, partial step
    const int64_t t = s0 + (int64_t)threadIdx.x * 4;
    if (t + 4 <= rw.len) {
      four(rw.base + t);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (t + k < rw.len) one(rw.base + t + k);
    }
  }
}

// ---------------------------------------------------------------- rows -> workgroups
// Workgroups are handed out in index order and, as measured, statically: round-robin over the
// eight XCDs and again over the shader engines inside one. With row b on workgroup b, row lengths
// that repeat with a short period (long and short rows interleaved by a length balancer, say) put
// all long rows on a fraction of the chip: with a quarter of the rows long, the per-token loss
// pass ran as slowly as if it had 2.9 times the tokens. Workgroup slot s therefore works on row
// row_of_slot(s): rows are permuted inside aligned blocks of 2^bits rows by a small bijective
// mix, XORed with a hash of the block's number so that no compute unit keeps meeting the same
// residue. Slot counts are rounded up to whole blocks; slots past n_rows are skipped. Blocks are
// 1/8 to 1/16 of the rows (8 to 256 rows), which bounds the skipped slots to about 12%.
__host__ __device__ inline int slot_bits(int64_t n_rows) {
  const int fl = n_rows > 0 ? 63 - __builtin_clzll((unsigned long long)n_rows) : 0;
  const int bits = fl - 3;
  return bits < 3 ? 3 : (bits > 8 ? 8 : bits);
}
__host__ __device__ inline int64_t row_slots(int64_t n_rows) {
  const int64_t blk = (int64_t)1 << slot_bits(n_rows);
  return (n_rows + blk - 1) & ~(blk - 1);
}
// `slot` counts inside one pass over the rows; `item` is the workgroup's global work index (equal
// to `slot` when a kernel makes a single pass) and only salts the hash.
__host__ __device__ __forceinline__ int64_t row_of_slot(int64_t slot, int64_t item, int bits) {
  const uint32_t mask = (1u << bits) - 1u;
  uint32_t x = (uint32_t)slot & mask;
  x = (x * 0x9Du) & mask;
  x ^= x >> ((bits + 1) >> 1);
  x = (x * 0x35u) & mask;
  uint32_t h = (uint32_t)(item >> bits) * 0x9E3779B1u;
  h ^= h >> 15;
  x ^= (h >> 7) & mask;
  return (slot & ~(int64_t)mask) | (int64_t)x;
}

// Grid for a kernel that walks `slots` work items with a grid-size stride.
inline unsigned slot_grid(int64_t slots, int64_t cap) {
  return (unsigned)(slots < cap ? (slots > 0 ? slots : 1) : cap);
}

inline int check_rows(const char* what, int64_t n_rows, int64_t n_cols, const void* mask, int mask_dtype) {
  if (n_rows < 0 || n_cols < 0)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: n_rows=%lld n_cols=%lld", what, (long long)n_rows, (long long)n_cols);
  if (!valid_mask_dtype(mask_dtype)) return fail(ORLHF_ERR_INVALID_ARG, "%s: unknown mask dtype %d", what, mask_dtype);
  if (mask_dtype != ORLHF_MASK_NONE && mask == nullptr && n_rows * n_cols > 0)
    return fail(ORLHF_ERR_INVALID_ARG, "%s: mask is NULL but mask dtype is %d", what, mask_dtype);
  return ORLHF_OK;
}

inline int flat_grid(int64_t n, int cap = 65536) {
  const int64_t g = (n + kBlock - 1) / kBlock;
  return (int)(g < cap ? (g > 0 ? g : 1) : cap);
}

}  // namespace orlhf
