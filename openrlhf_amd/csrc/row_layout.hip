// Row layout kernels for gfx950: between the reference's padded [B, A] per-token tensors (plus a
// mask) and the packed layout (flat tokens + cu_seqlens) that every per-token kernel of this
// library also accepts. Pure index work and copies: bit-exact, HBM/latency-bound.
//
//   row_extents   first / one-past-last non-zero column of every mask row
//   cu_seqlens    exclusive prefix sum of row lengths (one workgroup, chained 256-wide scans)
//   pack_rows     dst[cu[b] + j] = src[b, first[b] + j]
//   gather_rows   dst[cu[b] + j] = src[start[b] + j]: rows picked out of another packed array
//   pad_rows      dst[b, :] = fill, then the row's tokens on the left or on the right side
//   unpad         the non-zero positions of a [B, T] mask in row-major order (masks with holes too): their
//                 count per row, and per position its flat index, token, next token and rank in its row
//   pad_by_indices  the way back: zeros, then dst[indices[i]] = src[i]
#include "common.h"

namespace orlhf {

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void row_extents_kernel(const void* __restrict__ mask, int64_t n_rows,
                                                             int64_t n_cols, int64_t* __restrict__ first,
                                                             int64_t* __restrict__ end,
                                                             int64_t* __restrict__ length) {
  __shared__ long long lds_lo[kWavesPerBlock], lds_hi[kWavesPerBlock];
  const int slot_b = slot_bits(n_rows);
  for (int64_t slot = blockIdx.x; slot < row_slots(n_rows); slot += gridDim.x) {
    const int64_t b = row_of_slot(slot, slot, slot_b);
    if (b >= n_rows) continue;
    long long lo = n_cols, hi = 0;  // no non-zero column: first = n_cols, end = 0
    auto see = [&](bool nonzero, int64_t t) {
      if (nonzero) {
        lo = t < lo ? t : lo;
        hi = t + 1 > hi ? t + 1 : hi;
      }
    };
    if (MASK_DT == ORLHF_MASK_U8) {
      // byte masks: 16 columns per load between the row's 16-byte boundaries. A lane visits its
      // groups in rising order, so it only has to keep the first and the last group that held a
      // non-zero byte; the bytes themselves are looked at once, after the loop.
      const uint8_t* bytes = (const uint8_t*)mask + b * n_cols;
      int64_t head = (int64_t)((16 - ((uintptr_t)bytes & 15)) & 15);
      head = head < n_cols ? head : n_cols;
      const int64_t groups = (n_cols - head) / 16;
      for (int64_t t = threadIdx.x; t < head; t += kBlock) see(bytes[t] != 0, t);
      int64_t g_first = -1, g_last = -1;
      u32x4 w_first = {0u, 0u, 0u, 0u}, w_last = {0u, 0u, 0u, 0u};
#pragma unroll 4
      for (int64_t g = threadIdx.x; g < groups; g += kBlock) {
        const u32x4 w = *(const u32x4*)(bytes + head + g * 16);
        if ((w[0] | w[1] | w[2] | w[3]) != 0u) {
          if (g_first < 0) g_first = g, w_first = w;
          g_last = g, w_last = w;
        }
      }
      // bit 7 of every byte of nz(w) is set iff that byte of w is non-zero
      auto nz = [](uint32_t w) { return (((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u; };
      if (g_first >= 0) {
        int at = 0;
#pragma unroll
        for (int k = 3; k >= 0; --k)
          if (w_first[k] != 0u) at = 4 * k + (__builtin_ctz(nz(w_first[k])) >> 3);
        see(true, head + g_first * 16 + at);
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (w_last[k] != 0u) at = 4 * k + ((31 - __builtin_clz(nz(w_last[k]))) >> 3);
        see(true, head + g_last * 16 + at);
      }
      for (int64_t t = head + groups * 16 + threadIdx.x; t < n_cols; t += kBlock) see(bytes[t] != 0, t);
    } else {
#pragma unroll 8
      for (int64_t t = threadIdx.x; t < n_cols; t += kBlock) see(load_mask<MASK_DT>(mask, b * n_cols + t) != 0.0f, t);
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const long long l2 = __shfl_xor(lo, o, kWave), h2 = __shfl_xor(hi, o, kWave);
      lo = l2 < lo ? l2 : lo;
      hi = h2 > hi ? h2 : hi;
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds_lo[wave] = lo, lds_hi[wave] = hi;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        lo = lds_lo[w] < lo ? lds_lo[w] : lo;
        hi = lds_hi[w] > hi ? lds_hi[w] : hi;
      }
      if (first != nullptr) first[b] = lo;
      if (end != nullptr) end[b] = hi;
      if (length != nullptr) length[b] = hi > lo ? hi - lo : 0;
    }
    __syncthreads();
  }
}

// cu[0] = 0, cu[i+1] = cu[i] + lengths[i]. One workgroup of 1024 lanes walks the rows 1024 at a
// time (three barriers per step: 4 steps for 4096 rows instead of 16 with 256 lanes).
constexpr int kCuBlock = 1024;
constexpr int kCuWaves = kCuBlock / kWave;

__global__ __launch_bounds__(kCuBlock) void cu_seqlens_kernel(const int64_t* __restrict__ lengths, int64_t n_rows,
                                                              int64_t* __restrict__ cu) {
  __shared__ long long wave_tot[kCuWaves];
  __shared__ long long carry_s;
  if (threadIdx.x == 0) {
    carry_s = 0;
    cu[0] = 0;
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  for (int64_t base = 0; base < n_rows; base += kCuBlock) {
    const int64_t i = base + threadIdx.x;
    long long v = i < n_rows ? lengths[i] : 0;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {  // inclusive scan inside the wave
      const long long up = __shfl_up(v, o, kWave);
      if (lane >= o) v += up;
    }
    if (lane == kWave - 1) wave_tot[wave] = v;
    __syncthreads();
    long long before = carry_s;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    if (i < n_rows) cu[i + 1] = before + v;
    __syncthreads();
    if (threadIdx.x == kCuBlock - 1) carry_s = before + v;
    __syncthreads();
  }
}

// A workgroup moves copy_chunk<E>() consecutive columns of one row (16 KiB whatever the element). (row, chunk) items are numbered
// with the row varying fastest: workgroups go to the XCDs round-robin by index, and numbered
// chunk-fastest the chunks that hold tokens of short rows would pile up on a few XCDs.
constexpr int kCopyChunkBytes = 16384;
template <typename E>
constexpr int copy_chunk() { return kCopyChunkBytes / (int)sizeof(E); }

// 16 bytes of consecutive elements as one load or store. The type only promises the element's own
// alignment (source and destination rows start anywhere), which gfx950 global memory accepts.
typedef uint32_t u32x4_a1 __attribute__((ext_vector_type(4), aligned(1)));
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
template <int SIZE> struct Vec16Of { typedef u32x4_a4 type; };
template <> struct Vec16Of<1> { typedef u32x4_a1 type; };
template <> struct Vec16Of<2> { typedef u32x4_a2 type; };
template <typename E>
struct Vec16 {
  typedef typename Vec16Of<sizeof(E)>::type type;
  static constexpr int kElems = 16 / sizeof(E);
};

// PITCHED: the source is a padded [n_rows, n_cols] grid and `first` (nullable) the first column of
// each row. Otherwise the source is flat, `first[b]` is the element where output row b starts in
// it, and n_cols only bounds the row lengths (it sizes the grid).
template <typename E, bool PITCHED>
__global__ __launch_bounds__(kBlock) void pack_rows_kernel(const E* __restrict__ src, int64_t n_rows, int64_t n_cols,
                                                           const int64_t* __restrict__ first,
                                                           const int64_t* __restrict__ cu, E* __restrict__ dst) {
  constexpr int kCopyChunk = copy_chunk<E>();
  const int64_t chunks = (n_cols + kCopyChunk - 1) / kCopyChunk;
  const int64_t slots = row_slots(n_rows);
  const int slot_b = slot_bits(n_rows);
  for (int64_t w = blockIdx.x; w < slots * chunks; w += gridDim.x) {
    const int64_t chunk = w / slots, b = row_of_slot(w - chunk * slots, w, slot_b), j0 = chunk * kCopyChunk;
    if (b >= n_rows) continue;
    const int64_t start = cu[b], len = cu[b + 1] - start;
    if (j0 >= len) continue;
    const int64_t f = first != nullptr ? first[b] : 0;
    int64_t stop = j0 + kCopyChunk < len ? j0 + kCopyChunk : len;
    const int64_t bound = PITCHED ? n_cols - f : n_cols;  // the grid's columns / the stated longest row
    stop = stop < bound ? stop : bound;
    const E* in = PITCHED ? src + b * n_cols + f : src + f;
    E* out = dst + start;
    constexpr int kE = Vec16<E>::kElems;
    typedef typename Vec16<E>::type V;
    const int64_t groups = (stop - j0) / kE;
#pragma unroll 4
    for (int64_t g = threadIdx.x; g < groups; g += kBlock) *(V*)(out + j0 + g * kE) = __builtin_nontemporal_load((const V*)(in + j0 + g * kE));
    for (int64_t j = j0 + groups * kE + threadIdx.x; j < stop; j += kBlock) out[j] = in[j];
  }
}

// Several [n_rows, n_cols] fields packed by ONE launch: a workgroup takes a stretch of kMultiCols
// columns of one row and copies it out of every field in turn (what a rollout batch needs: four to ten
// per-token fields share one mask). Items are numbered row-major, the stretches of a row rotated by
// the row number: the workgroups that run together read and write neighbouring memory in every
// field, and the stretches past the ends of short rows do not all fall on the same XCDs.
constexpr int kMaxPackFields = 8;
constexpr int kMultiCols = 4096;
struct PackFields {
  const void* src[kMaxPackFields];
  void* dst[kMaxPackFields];
  int elem_bytes[kMaxPackFields];
  int n;
};

template <typename E>
__device__ __forceinline__ void copy_stretch(const E* __restrict__ in, E* __restrict__ out, int64_t j0, int64_t stop) {
  constexpr int kE = Vec16<E>::kElems;
  typedef typename Vec16<E>::type V;
  const int64_t groups = (stop - j0) / kE;
#pragma unroll 4
  for (int64_t g = threadIdx.x; g < groups; g += kBlock) *(V*)(out + j0 + g * kE) = __builtin_nontemporal_load((const V*)(in + j0 + g * kE));
  for (int64_t j = j0 + groups * kE + threadIdx.x; j < stop; j += kBlock) out[j] = in[j];
}

__global__ __launch_bounds__(kBlock) void pack_rows_multi_kernel(PackFields f, int64_t n_rows, int64_t n_cols,
                                                                 const int64_t* __restrict__ first,
                                                                 const int64_t* __restrict__ cu) {
  const int64_t chunks = (n_cols + kMultiCols - 1) / kMultiCols;
  // rows fastest, as in the one-field kernel (row-major numbering of the items measured 6 % slower here)
  const int64_t slots = row_slots(n_rows);
  const int slot_b = slot_bits(n_rows);
  for (int64_t w = blockIdx.x; w < slots * chunks; w += gridDim.x) {
    const int64_t chunk = w / slots, b = row_of_slot(w - chunk * slots, w, slot_b);
    if (b >= n_rows) continue;
    const int64_t j0 = chunk * kMultiCols;
    const int64_t start = cu[b], len = cu[b + 1] - start;
    if (j0 >= len) continue;
    const int64_t fst = first != nullptr ? first[b] : 0;
    int64_t stop = j0 + kMultiCols < len ? j0 + kMultiCols : len;
    stop = stop < n_cols - fst ? stop : n_cols - fst;
    const int64_t in0 = b * n_cols + fst;
#pragma unroll 1
    for (int i = 0; i < f.n; ++i) {
      switch (f.elem_bytes[i]) {
        case 1: copy_stretch((const uint8_t*)f.src[i] + in0, (uint8_t*)f.dst[i] + start, j0, stop); break;
        case 2: copy_stretch((const uint16_t*)f.src[i] + in0, (uint16_t*)f.dst[i] + start, j0, stop); break;
        case 4: copy_stretch((const uint32_t*)f.src[i] + in0, (uint32_t*)f.dst[i] + start, j0, stop); break;
        default: copy_stretch((const uint64_t*)f.src[i] + in0, (uint64_t*)f.dst[i] + start, j0, stop); break;
      }
    }
  }
}

template <typename E>
__global__ __launch_bounds__(kBlock) void pad_rows_kernel(const E* __restrict__ src, const int64_t* __restrict__ cu,
                                                          int64_t n_rows, int64_t n_cols, int left, E fill,
                                                          E* __restrict__ dst) {
  constexpr int kCopyChunk = copy_chunk<E>();
  const int64_t chunks = (n_cols + kCopyChunk - 1) / kCopyChunk;
  for (int64_t w = blockIdx.x; w < n_rows * chunks; w += gridDim.x) {
    const int64_t chunk = w / n_rows, b = w - chunk * n_rows, t0 = chunk * kCopyChunk;
    const int64_t start = cu[b];
    int64_t len = cu[b + 1] - start;
    len = len < n_cols ? len : n_cols;  // a longer row is cut at n_cols
    const int64_t shift = left ? n_cols - len : 0;  // column of the row's first token
    const int64_t stop = t0 + kCopyChunk < n_cols ? t0 + kCopyChunk : n_cols;
    E* out = dst + b * n_cols;
    constexpr int kE = Vec16<E>::kElems;
    typedef typename Vec16<E>::type V;
    E fill_e[kE];
#pragma unroll
    for (int k = 0; k < kE; ++k) fill_e[k] = fill;
    const V fill_v = __builtin_bit_cast(V, fill_e);
    const int64_t groups = (stop - t0) / kE;
#pragma unroll 2
    for (int64_t g = threadIdx.x; g < groups; g += kBlock) {
      const int64_t t = t0 + g * kE;
      if (t >= shift && t + kE <= shift + len) {  // all of the group's columns hold tokens
        *(V*)(out + t) = __builtin_nontemporal_load((const V*)(src + start + (t - shift)));
      } else if (t + kE <= shift || t >= shift + len) {  // all padding
        *(V*)(out + t) = fill_v;
      } else {
#pragma unroll
        for (int k = 0; k < kE; ++k)
          out[t + k] = (t + k >= shift && t + k < shift + len) ? src[start + (t + k - shift)] : fill;
      }
    }
    for (int64_t t = t0 + groups * kE + threadIdx.x; t < stop; t += kBlock)
      out[t] = (t >= shift && t < shift + len) ? src[start + (t - shift)] : fill;
  }
}

// Non-zero columns of mask row b in rising order. A workgroup walks its row in tiles of
// kUnpadCols * kBlock columns, kUnpadCols consecutive columns per lane; a lane's rank among the
// row's non-zero columns is (non-zeros of earlier tiles) + (those of earlier waves) + (wave scan).
// COUNT_ONLY leaves the row's count; otherwise position r of row b goes to slot cu[b] + r of every
// output that is asked for: its flat index b * n_cols + t, sequences[b, t],
// sequences[b, (t + 1) mod n_cols] and r. A lane whose columns are all non-zero (the inside of an
// attended span: almost every lane that writes at all) moves its tokens with 16-byte loads and
// stores.
constexpr int kUnpadCols = 8;

template <int MASK_DT, bool COUNT_ONLY>
__global__ __launch_bounds__(kBlock) void unpad_rows_kernel(const int64_t* __restrict__ sequences,
                                                            const void* __restrict__ mask, int64_t n_rows, int64_t n_cols,
                                                            const int64_t* __restrict__ cu, int64_t capacity,
                                                            int64_t* __restrict__ counts, int32_t* __restrict__ chunk_counts,
                                                            int64_t* __restrict__ indices, int64_t* __restrict__ packed,
                                                            int64_t* __restrict__ rolled, int64_t* __restrict__ position) {
  __shared__ int wave_tot[2][kWavesPerBlock];  // alternating slots: one barrier per tile
  const int64_t n_chunks = (n_cols + kUnpadCols * kBlock - 1) / (kUnpadCols * kBlock);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int par = 0;
  for (int64_t b = blockIdx.x; b < n_rows; b += gridDim.x) {
    const int64_t out0 = COUNT_ONLY ? 0 : cu[b];
    int64_t run = 0;  // non-zero columns of the row before this tile
    for (int64_t t0 = 0; t0 < n_cols; t0 += kUnpadCols * kBlock, par ^= 1) {
      const int64_t t = t0 + kUnpadCols * (int64_t)threadIdx.x;
      uint32_t nz = 0;  // bit k: column t + k is inside the row and non-zero
      if (t + kUnpadCols <= n_cols) {  // whole group inside the row
        float m[kUnpadCols];
#pragma unroll
        for (int q = 0; q < kUnpadCols / 4; ++q) load_mask4<MASK_DT, false>(mask, b * n_cols + t + 4 * q, m + 4 * q);
#pragma unroll
        for (int k = 0; k < kUnpadCols; ++k) nz |= m[k] != 0.0f ? 1u << k : 0u;
      } else {
#pragma unroll
        for (int k = 0; k < kUnpadCols; ++k)
          nz |= (t + k < n_cols && load_mask<MASK_DT>(mask, b * n_cols + t + k) != 0.0f) ? 1u << k : 0u;
      }
      const int c = __builtin_popcount(nz);
      int incl = c;
#pragma unroll
      for (int o = 1; o < kWave; o <<= 1) {
        const int up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
      }
      if (lane == kWave - 1) wave_tot[par][wave] = incl;
      __syncthreads();
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        const int v = wave_tot[par][w];
        before += w < wave ? v : 0;
        total += v;
      }
      constexpr int kWaveCols = kUnpadCols * kWave;
      const bool wave_dense = !COUNT_ONLY && __all(nz == (1u << kUnpadCols) - 1u) &&
                              out0 + run + before + kWaveCols <= capacity;
      if (wave_dense) {
        // the wave's 512 columns are 512 consecutive slots: lanes take them two at a time, interleaved,
        // so that every load and store of the wave covers 1 KiB of consecutive memory
        const int64_t col0 = t0 + (int64_t)wave * kWaveCols, at0 = b * n_cols + col0, dst0 = out0 + run + before;
#pragma unroll
        for (int j = 0; j < kWaveCols / (2 * kWave); ++j) {
          const int64_t off = 2 * kWave * j + 2 * lane;
          if (indices != nullptr) *(i64x2e*)(indices + dst0 + off) = i64x2{at0 + off, at0 + off + 1};
          if (position != nullptr) *(i64x2e*)(position + dst0 + off) = i64x2{run + before + off, run + before + off + 1};
          if (packed != nullptr || rolled != nullptr) {
            const i64x2 v = *(const i64x2e*)(sequences + at0 + off);
            if (packed != nullptr) *(i64x2e*)(packed + dst0 + off) = v;
            if (rolled != nullptr) {
              const int64_t after = sequences[col0 + off + 2 == n_cols ? b * n_cols : at0 + off + 2];
              *(i64x2e*)(rolled + dst0 + off) = i64x2{v[1], after};
            }
          }
        }
      } else if (!COUNT_ONLY && c > 0) {
        int64_t r = run + before + incl - c;
        const int64_t at0 = b * n_cols + t, dst0 = out0 + r;
        if (nz == (1u << kUnpadCols) - 1u && dst0 + kUnpadCols <= capacity) {
          int64_t tok[kUnpadCols + 1];
          if (packed != nullptr || rolled != nullptr) {
#pragma unroll
            for (int q = 0; q < kUnpadCols / 2; ++q) {
              const i64x2 v = *(const i64x2e*)(sequences + at0 + 2 * q);
              tok[2 * q] = v[0];
              tok[2 * q + 1] = v[1];
            }
            tok[kUnpadCols] = rolled != nullptr ? sequences[t + kUnpadCols == n_cols ? b * n_cols : at0 + kUnpadCols] : 0;
          }
#pragma unroll
          for (int q = 0; q < kUnpadCols / 2; ++q) {
            if (indices != nullptr) *(i64x2e*)(indices + dst0 + 2 * q) = i64x2{at0 + 2 * q, at0 + 2 * q + 1};
            if (packed != nullptr) *(i64x2e*)(packed + dst0 + 2 * q) = i64x2{tok[2 * q], tok[2 * q + 1]};
            if (rolled != nullptr) *(i64x2e*)(rolled + dst0 + 2 * q) = i64x2{tok[2 * q + 1], tok[2 * q + 2]};
            if (position != nullptr) *(i64x2e*)(position + dst0 + 2 * q) = i64x2{r + 2 * q, r + 2 * q + 1};
          }
        } else {
#pragma unroll
          for (int k = 0; k < kUnpadCols; ++k) {
            const bool on = (nz >> k) & 1u;
            if (on && out0 + r < capacity) {  // slots past the outputs' stated size are dropped
              const int64_t at = at0 + k, dst = out0 + r;
              if (indices != nullptr) indices[dst] = at;
              if (packed != nullptr) packed[dst] = sequences[at];
              if (rolled != nullptr) rolled[dst] = sequences[t + k + 1 == n_cols ? b * n_cols : at + 1];
              if (position != nullptr) position[dst] = r;
            }
            r += on ? 1 : 0;
          }
        }
      }
      if (COUNT_ONLY && chunk_counts != nullptr && threadIdx.x == 0) chunk_counts[b * n_chunks + t0 / (kUnpadCols * kBlock)] = total;
      run += total;
    }
    if (COUNT_ONLY && threadIdx.x == 0) counts[b] = run;
  }
}

// The same outputs with one workgroup per (row, tile of kUnpadCols * kBlock columns) instead of one
// per row: chunk_counts[b][tile] (from the counting pass) gives every tile its first slot without
// waiting for the tiles before it, a tile without non-zero columns costs one load of its count, and
// a tile whose columns are all non-zero (the inside of an attended span: all but one or two tiles
// of a row) does not read the mask at all.
// One tile per workgroup: with 2, 3 or 4 consecutive tiles of a row per workgroup the same launch
// (4096 x 16385 cells, half attended, all four outputs) took 0.277, 0.291 and 0.299 ms against 0.272.

template <int MASK_DT>
__global__ __launch_bounds__(kBlock) void unpad_tiles_kernel(const int64_t* __restrict__ sequences,
                                                             const void* __restrict__ mask, int64_t n_rows, int64_t n_cols,
                                                             const int64_t* __restrict__ cu,
                                                             const int32_t* __restrict__ chunk_counts, int64_t capacity,
                                                             int64_t* __restrict__ indices, int64_t* __restrict__ packed,
                                                             int64_t* __restrict__ rolled, int64_t* __restrict__ position) {
  constexpr int kTileCols = kUnpadCols * kBlock, kWaveCols = kUnpadCols * kWave;
  __shared__ int wave_tot[kWavesPerBlock];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t n_chunks = (n_cols + kTileCols - 1) / kTileCols;
  for (int64_t w = blockIdx.x; w < n_rows * n_chunks; w += gridDim.x) {
    // row-major: the workgroups that run at the same time write neighbouring stretches of every
    // output (DRAM pages stay open); the tiles of a row are taken in an order rotated by the row
    // number, so that the tiles past the ends of short rows do not all fall on the same XCDs
    const int64_t b = w / n_chunks;
    int64_t ch = (w - b * n_chunks) + b % n_chunks;
    ch = ch >= n_chunks ? ch - n_chunks : ch;
    const int32_t* cc = chunk_counts + b * n_chunks;
    const int c_tile = cc[ch];
    if (c_tile == 0) continue;
    int64_t run = 0;  // non-zero columns of the row before this tile (every wave sums them for itself)
    for (int64_t j = lane; j < ch; j += kWave) run += cc[j];
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) run += __shfl_xor(run, o, kWave);
    const int64_t out0 = cu[b];
    const int64_t t0 = ch * kTileCols;
    // the wave's 512 columns as 512 consecutive slots: lanes take them two at a time, interleaved,
    // so that every load and store of the wave covers 1 KiB of consecutive memory
    auto dense_wave = [&](int64_t before) {
      constexpr int kIter = kWaveCols / (2 * kWave);
      const int64_t col0 = t0 + (int64_t)wave * kWaveCols, at0 = b * n_cols + col0, dst0 = out0 + run + before;
      i64x2 v[kIter];
      int64_t past = 0;  // the token after the wave's last column (lane 63 needs it for the rolled output)
      if (packed != nullptr || rolled != nullptr) {
#pragma unroll
        for (int j = 0; j < kIter; ++j) v[j] = __builtin_nontemporal_load((const i64x2e*)(sequences + at0 + 2 * kWave * j + 2 * lane));
        if (rolled != nullptr && lane == kWave - 1) past = sequences[col0 + kWaveCols == n_cols ? b * n_cols : at0 + kWaveCols];
      }
#pragma unroll
      for (int j = 0; j < kIter; ++j) {
        const int64_t off = 2 * kWave * j + 2 * lane;
        if (indices != nullptr) *(i64x2e*)(indices + dst0 + off) = i64x2{at0 + off, at0 + off + 1};
        if (position != nullptr) *(i64x2e*)(position + dst0 + off) = i64x2{run + before + off, run + before + off + 1};
        if (packed != nullptr) *(i64x2e*)(packed + dst0 + off) = v[j];
        if (rolled != nullptr) {
          // the token after this lane's pair is the next lane's first one (the first lane's of the next
          // step for the last lane): no second load of lines the streaming load did not keep
          int64_t after = __shfl_down(v[j][0], 1, kWave);
          const int64_t wrap = j + 1 < kIter ? __shfl(v[j + 1 < kIter ? j + 1 : j][0], 0, kWave) : past;
          after = lane == kWave - 1 ? wrap : after;
          *(i64x2e*)(rolled + dst0 + off) = i64x2{v[j][1], after};  // (non-temporal stores: one output alone 20 % faster, all four 8 % slower)
        }
      }
    };
    if (c_tile == kTileCols && out0 + run + kTileCols <= capacity) {  // all columns attended: the mask is not read
      dense_wave((int64_t)wave * kWaveCols);
      continue;
    }
    const int64_t t = t0 + kUnpadCols * (int64_t)threadIdx.x;
    uint32_t nz = 0;  // bit k: column t + k is inside the row and non-zero
    if (t + kUnpadCols <= n_cols) {
      float m[kUnpadCols];
#pragma unroll
      for (int q = 0; q < kUnpadCols / 4; ++q) load_mask4<MASK_DT, false>(mask, b * n_cols + t + 4 * q, m + 4 * q);
#pragma unroll
      for (int k = 0; k < kUnpadCols; ++k) nz |= m[k] != 0.0f ? 1u << k : 0u;
    } else {
#pragma unroll
      for (int k = 0; k < kUnpadCols; ++k)
        nz |= (t + k < n_cols && load_mask<MASK_DT>(mask, b * n_cols + t + k) != 0.0f) ? 1u << k : 0u;
    }
    const int c = __builtin_popcount(nz);
    int incl = c;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(incl, o, kWave);
      if (lane >= o) incl += up;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int before = 0;
#pragma unroll
    for (int w2 = 0; w2 < kWavesPerBlock; ++w2) before += w2 < wave ? wave_tot[w2] : 0;
    __syncthreads();  // wave_tot is free for the workgroup's next item
    if (__all(nz == (1u << kUnpadCols) - 1u) && out0 + run + before + kWaveCols <= capacity) {
      dense_wave(before);
    } else if (c > 0) {
      int64_t r = run + before + incl - c;
      const int64_t at0 = b * n_cols + t, dst0 = out0 + r;
      if (nz == (1u << kUnpadCols) - 1u && dst0 + kUnpadCols <= capacity) {
        int64_t tok[kUnpadCols + 1];
        if (packed != nullptr || rolled != nullptr) {
#pragma unroll
          for (int q = 0; q < kUnpadCols / 2; ++q) {
            const i64x2 v = *(const i64x2e*)(sequences + at0 + 2 * q);
            tok[2 * q] = v[0];
            tok[2 * q + 1] = v[1];
          }
          tok[kUnpadCols] = rolled != nullptr ? sequences[t + kUnpadCols == n_cols ? b * n_cols : at0 + kUnpadCols] : 0;
        }
#pragma unroll
        for (int q = 0; q < kUnpadCols / 2; ++q) {
          if (indices != nullptr) *(i64x2e*)(indices + dst0 + 2 * q) = i64x2{at0 + 2 * q, at0 + 2 * q + 1};
          if (packed != nullptr) *(i64x2e*)(packed + dst0 + 2 * q) = i64x2{tok[2 * q], tok[2 * q + 1]};
          if (rolled != nullptr) *(i64x2e*)(rolled + dst0 + 2 * q) = i64x2{tok[2 * q + 1], tok[2 * q + 2]};
          if (position != nullptr) *(i64x2e*)(position + dst0 + 2 * q) = i64x2{r + 2 * q, r + 2 * q + 1};
        }
      } else {
#pragma unroll
        for (int k = 0; k < kUnpadCols; ++k) {
          const bool on = (nz >> k) & 1u;
          if (on && out0 + r < capacity) {  // slots past the outputs' stated size are dropped
            const int64_t at = at0 + k, dst = out0 + r;
            if (indices != nullptr) indices[dst] = at;
            if (packed != nullptr) packed[dst] = sequences[at];
            if (rolled != nullptr) rolled[dst] = sequences[t + k + 1 == n_cols ? b * n_cols : at + 1];
            if (position != nullptr) position[dst] = r;
          }
          r += on ? 1 : 0;
        }
      }
    }
  }
}

// dst[indices[i] * inner + j] = src[i * inner + j]; an index outside [0, n_dst) is skipped.
template <typename E>
__global__ __launch_bounds__(kBlock) void scatter_index_kernel(const E* __restrict__ src, const int64_t* __restrict__ indices,
                                                               int64_t n, int64_t inner, int64_t n_dst, E* __restrict__ dst) {
  const int64_t total = n * inner;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total; e += (int64_t)gridDim.x * kBlock) {
    const int64_t i = e / inner, j = e - i * inner, to = indices[i];
    if ((uint64_t)to < (uint64_t)n_dst) dst[to * inner + j] = src[e];
  }
}

// dst[i * inner + j] = src[indices[i] * inner + j] (flash-attn's index_first_axis): V = the widest
// unit (1 to 16 bytes) that divides a row and both bases, `units` of them per row; an index outside
// [0, n_src) gives zeros.
template <typename V>
__global__ __launch_bounds__(kBlock) void gather_index_kernel(const V* __restrict__ src, const int64_t* __restrict__ indices,
                                                              int64_t n, int64_t units, int64_t n_src, V* __restrict__ dst) {
  const int64_t total = n * units;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total; e += (int64_t)gridDim.x * kBlock) {
    const int64_t i = e / units, j = e - i * units, from = indices[i];
    V v{};
    if ((uint64_t)from < (uint64_t)n_src) v = src[from * units + j];
    dst[e] = v;
  }
}

__global__ __launch_bounds__(kBlock) void zero_bytes_kernel(char* __restrict__ dst, int64_t bytes) {
  const int64_t groups = bytes / 16;  // dst is 16-byte aligned (checked by the caller)
  for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < groups; g += (int64_t)gridDim.x * kBlock)
    *(u32x4*)(dst + g * 16) = u32x4{0u, 0u, 0u, 0u};
  for (int64_t i = groups * 16 + (int64_t)blockIdx.x * kBlock + threadIdx.x; i < bytes; i += (int64_t)gridDim.x * kBlock) dst[i] = 0;
}

static inline unsigned copy_grid(int64_t n_rows, int64_t n_cols, int elem_bytes) {
  const int64_t chunk = kCopyChunkBytes / elem_bytes;
  const int64_t chunks = (n_cols + chunk - 1) / chunk;
  return slot_grid(row_slots(n_rows) * chunks, 262144);
}

}  // namespace orlhf

using namespace orlhf;

extern "C" int orlhf_row_extents(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols, int64_t* first,
                                 int64_t* end, int64_t* length, orlhf_stream_t stream) {
  if (int rc = check_rows("row_extents", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mask_dtype != ORLHF_MASK_NONE, "row_extents: needs a mask");
  if (n_rows == 0) return ORLHF_OK;
  const dim3 grid(slot_grid(row_slots(n_rows), 65536)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  switch (mask_dtype) {
    case ORLHF_MASK_U8:
      hipLaunchKernelGGL(row_extents_kernel<ORLHF_MASK_U8>, grid, block, 0, s, mask, n_rows, n_cols, first, end, length);
      break;
    case ORLHF_MASK_F32:
      hipLaunchKernelGGL(row_extents_kernel<ORLHF_MASK_F32>, grid, block, 0, s, mask, n_rows, n_cols, first, end, length);
      break;
    default:
      hipLaunchKernelGGL(row_extents_kernel<ORLHF_MASK_I64>, grid, block, 0, s, mask, n_rows, n_cols, first, end, length);
      break;
  }
  ORLHF_CHECK_LAUNCH("orlhf_row_extents");
  return ORLHF_OK;
}

extern "C" int orlhf_cu_seqlens(const int64_t* lengths, int64_t n_rows, int64_t* cu_seqlens, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0, "cu_seqlens: n_rows=%lld", (long long)n_rows);
  ORLHF_CHECK_ARG(cu_seqlens != nullptr && (lengths != nullptr || n_rows == 0), "cu_seqlens: NULL argument");
  hipLaunchKernelGGL(cu_seqlens_kernel, dim3(1), dim3(kCuBlock), 0, (hipStream_t)stream, lengths, n_rows, cu_seqlens);
  ORLHF_CHECK_LAUNCH("orlhf_cu_seqlens");
  return ORLHF_OK;
}

extern "C" int orlhf_pack_rows(const void* src, int elem_bytes, int64_t n_rows, int64_t n_cols, const int64_t* first,
                               const int64_t* cu_seqlens, void* dst, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && n_cols >= 0, "pack_rows: n_rows=%lld n_cols=%lld", (long long)n_rows, (long long)n_cols);
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(src != nullptr && dst != nullptr && cu_seqlens != nullptr, "pack_rows: NULL argument");
  ORLHF_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                  "row layout: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  const dim3 grid(copy_grid(n_rows, n_cols, elem_bytes)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL((pack_rows_kernel<uint8_t, true>), grid, block, 0, s, (const uint8_t*)src, n_rows, n_cols, first, cu_seqlens, (uint8_t*)dst); break;
    case 2: hipLaunchKernelGGL((pack_rows_kernel<uint16_t, true>), grid, block, 0, s, (const uint16_t*)src, n_rows, n_cols, first, cu_seqlens, (uint16_t*)dst); break;
    case 4: hipLaunchKernelGGL((pack_rows_kernel<uint32_t, true>), grid, block, 0, s, (const uint32_t*)src, n_rows, n_cols, first, cu_seqlens, (uint32_t*)dst); break;
    case 8: hipLaunchKernelGGL((pack_rows_kernel<uint64_t, true>), grid, block, 0, s, (const uint64_t*)src, n_rows, n_cols, first, cu_seqlens, (uint64_t*)dst); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "pack_rows: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  }
  ORLHF_CHECK_LAUNCH("orlhf_pack_rows");
  return ORLHF_OK;
}

extern "C" int orlhf_pack_rows_multi(const orlhf_pack_field* fields, int n_fields, int64_t n_rows, int64_t n_cols,
                                     const int64_t* first, const int64_t* cu_seqlens, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && n_cols >= 0 && n_fields >= 0, "pack_rows_multi: n_rows=%lld n_cols=%lld n_fields=%d",
                  (long long)n_rows, (long long)n_cols, n_fields);
  if (n_rows * n_cols == 0 || n_fields == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(fields != nullptr && cu_seqlens != nullptr, "pack_rows_multi: NULL argument");
  hipStream_t s = (hipStream_t)stream;
  const int64_t chunks = (n_cols + kMultiCols - 1) / kMultiCols;
  const dim3 grid(slot_grid(row_slots(n_rows) * chunks, 1 << 20)), block(kBlock);
  for (int at = 0; at < n_fields; at += kMaxPackFields) {  // eight fields per launch: they travel in the kernel arguments
    PackFields f;
    f.n = n_fields - at < kMaxPackFields ? n_fields - at : kMaxPackFields;
    for (int i = 0; i < f.n; ++i) {
      const orlhf_pack_field& g = fields[at + i];
      ORLHF_CHECK_ARG(g.src != nullptr && g.dst != nullptr, "pack_rows_multi: field %d has a NULL pointer", at + i);
      ORLHF_CHECK_ARG(g.elem_bytes == 1 || g.elem_bytes == 2 || g.elem_bytes == 4 || g.elem_bytes == 8,
                      "row layout: element size %d (1, 2, 4 or 8 bytes)", g.elem_bytes);
      f.src[i] = g.src, f.dst[i] = g.dst, f.elem_bytes[i] = g.elem_bytes;
    }
    hipLaunchKernelGGL(pack_rows_multi_kernel, grid, block, 0, s, f, n_rows, n_cols, first, cu_seqlens);
    ORLHF_CHECK_LAUNCH("orlhf_pack_rows_multi");
  }
  return ORLHF_OK;
}

extern "C" int orlhf_gather_rows(const void* src, int elem_bytes, int64_t n_rows, int64_t max_len,
                                 const int64_t* src_start, const int64_t* cu_seqlens, void* dst,
                                 orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && max_len >= 0, "gather_rows: n_rows=%lld max_len=%lld", (long long)n_rows, (long long)max_len);
  if (n_rows * max_len == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(src != nullptr && dst != nullptr && cu_seqlens != nullptr && src_start != nullptr,
                  "gather_rows: NULL argument");
  ORLHF_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                  "row layout: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  const dim3 grid(copy_grid(n_rows, max_len, elem_bytes)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL((pack_rows_kernel<uint8_t, false>), grid, block, 0, s, (const uint8_t*)src, n_rows, max_len, src_start, cu_seqlens, (uint8_t*)dst); break;
    case 2: hipLaunchKernelGGL((pack_rows_kernel<uint16_t, false>), grid, block, 0, s, (const uint16_t*)src, n_rows, max_len, src_start, cu_seqlens, (uint16_t*)dst); break;
    case 4: hipLaunchKernelGGL((pack_rows_kernel<uint32_t, false>), grid, block, 0, s, (const uint32_t*)src, n_rows, max_len, src_start, cu_seqlens, (uint32_t*)dst); break;
    default: hipLaunchKernelGGL((pack_rows_kernel<uint64_t, false>), grid, block, 0, s, (const uint64_t*)src, n_rows, max_len, src_start, cu_seqlens, (uint64_t*)dst); break;
  }
  ORLHF_CHECK_LAUNCH("orlhf_gather_rows");
  return ORLHF_OK;
}

extern "C" int orlhf_pad_rows(const void* src, int elem_bytes, const int64_t* cu_seqlens, int64_t n_rows,
                              int64_t n_cols, int left_side, uint64_t fill_bits, void* dst, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n_rows >= 0 && n_cols >= 0, "pad_rows: n_rows=%lld n_cols=%lld", (long long)n_rows, (long long)n_cols);
  if (n_rows * n_cols == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(dst != nullptr && cu_seqlens != nullptr, "pad_rows: NULL argument");
  ORLHF_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                  "row layout: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  const dim3 grid(copy_grid(n_rows, n_cols, elem_bytes)), block(kBlock);
  hipStream_t s = (hipStream_t)stream;
  const int left = left_side != 0;
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL(pad_rows_kernel<uint8_t>, grid, block, 0, s, (const uint8_t*)src, cu_seqlens, n_rows, n_cols, left, (uint8_t)fill_bits, (uint8_t*)dst); break;
    case 2: hipLaunchKernelGGL(pad_rows_kernel<uint16_t>, grid, block, 0, s, (const uint16_t*)src, cu_seqlens, n_rows, n_cols, left, (uint16_t)fill_bits, (uint16_t*)dst); break;
    case 4: hipLaunchKernelGGL(pad_rows_kernel<uint32_t>, grid, block, 0, s, (const uint32_t*)src, cu_seqlens, n_rows, n_cols, left, (uint32_t)fill_bits, (uint32_t*)dst); break;
    case 8: hipLaunchKernelGGL(pad_rows_kernel<uint64_t>, grid, block, 0, s, (const uint64_t*)src, cu_seqlens, n_rows, n_cols, left, (uint64_t)fill_bits, (uint64_t*)dst); break;
    default: return fail(ORLHF_ERR_INVALID_ARG, "pad_rows: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  }
  ORLHF_CHECK_LAUNCH("orlhf_pad_rows");
  return ORLHF_OK;
}

template <bool COUNT_ONLY>
static int launch_unpad(const int64_t* sequences, const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                        const int64_t* cu, int64_t capacity, int64_t* counts, int32_t* chunk_counts, int64_t* indices,
                        int64_t* packed, int64_t* rolled, int64_t* position, hipStream_t s) {
  const dim3 grid(slot_grid(n_rows, 65536)), block(kBlock);
  switch (mask_dtype) {
    case ORLHF_MASK_U8:
      hipLaunchKernelGGL((unpad_rows_kernel<ORLHF_MASK_U8, COUNT_ONLY>), grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, capacity, counts, chunk_counts, indices, packed, rolled, position);
      break;
    case ORLHF_MASK_F32:
      hipLaunchKernelGGL((unpad_rows_kernel<ORLHF_MASK_F32, COUNT_ONLY>), grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, capacity, counts, chunk_counts, indices, packed, rolled, position);
      break;
    default:
      hipLaunchKernelGGL((unpad_rows_kernel<ORLHF_MASK_I64, COUNT_ONLY>), grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, capacity, counts, chunk_counts, indices, packed, rolled, position);
      break;
  }
  return ORLHF_OK;
}

static void launch_unpad_tiles(const int64_t* sequences, const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols,
                               const int64_t* cu, const int32_t* chunk_counts, int64_t capacity, int64_t* indices,
                               int64_t* packed, int64_t* rolled, int64_t* position, hipStream_t s) {
  const int64_t n_chunks = (n_cols + ORLHF_UNPAD_TILE - 1) / ORLHF_UNPAD_TILE;
  const dim3 grid(slot_grid(n_rows * n_chunks, 1 << 20)), block(kBlock);
  switch (mask_dtype) {
    case ORLHF_MASK_U8:
      hipLaunchKernelGGL(unpad_tiles_kernel<ORLHF_MASK_U8>, grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, chunk_counts, capacity, indices, packed, rolled, position);
      break;
    case ORLHF_MASK_F32:
      hipLaunchKernelGGL(unpad_tiles_kernel<ORLHF_MASK_F32>, grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, chunk_counts, capacity, indices, packed, rolled, position);
      break;
    default:
      hipLaunchKernelGGL(unpad_tiles_kernel<ORLHF_MASK_I64>, grid, block, 0, s, sequences, mask, n_rows, n_cols, cu, chunk_counts, capacity, indices, packed, rolled, position);
      break;
  }
}

static_assert(ORLHF_UNPAD_TILE == kUnpadCols * kBlock, "the header states the tile of the unpadding kernels");

extern "C" int orlhf_mask_row_counts(const void* mask, int mask_dtype, int64_t n_rows, int64_t n_cols, int64_t* counts,
                                     int32_t* tile_counts, orlhf_stream_t stream) {
  if (int rc = check_rows("mask_row_counts", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mask_dtype != ORLHF_MASK_NONE, "mask_row_counts: needs a mask");
  if (n_rows == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(counts != nullptr, "mask_row_counts: counts is NULL");
  launch_unpad<true>(nullptr, mask, mask_dtype, n_rows, n_cols, nullptr, 0, counts, tile_counts, nullptr, nullptr, nullptr,
                     nullptr, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_mask_row_counts");
  return ORLHF_OK;
}

extern "C" int orlhf_unpad_sequences(const int64_t* sequences, const void* mask, int mask_dtype, int64_t n_rows,
                                     int64_t n_cols, const int64_t* cu_seqlens, const int32_t* tile_counts,
                                     int64_t capacity, int64_t* indices, int64_t* packed_sequences,
                                     int64_t* rolled_sequences, int64_t* position_ids, orlhf_stream_t stream) {
  if (int rc = check_rows("unpad_sequences", n_rows, n_cols, mask, mask_dtype)) return rc;
  ORLHF_CHECK_ARG(mask_dtype != ORLHF_MASK_NONE, "unpad_sequences: needs a mask");
  ORLHF_CHECK_ARG(capacity >= 0, "unpad_sequences: capacity=%lld", (long long)capacity);
  if (n_rows * n_cols == 0 || capacity == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(cu_seqlens != nullptr, "unpad_sequences: cu_seqlens is NULL");
  ORLHF_CHECK_ARG(indices != nullptr || packed_sequences != nullptr || rolled_sequences != nullptr || position_ids != nullptr,
                  "unpad_sequences: nothing to compute");
  ORLHF_CHECK_ARG(sequences != nullptr || (packed_sequences == nullptr && rolled_sequences == nullptr),
                  "unpad_sequences: sequences is NULL");
  if (tile_counts != nullptr)
    launch_unpad_tiles(sequences, mask, mask_dtype, n_rows, n_cols, cu_seqlens, tile_counts, capacity, indices, packed_sequences,
                       rolled_sequences, position_ids, (hipStream_t)stream);
  else
    launch_unpad<false>(sequences, mask, mask_dtype, n_rows, n_cols, cu_seqlens, capacity, nullptr, nullptr, indices,
                        packed_sequences, rolled_sequences, position_ids, (hipStream_t)stream);
  ORLHF_CHECK_LAUNCH("orlhf_unpad_sequences");
  return ORLHF_OK;
}

extern "C" int orlhf_pad_by_indices(const void* src, int elem_bytes, int64_t n, int64_t inner, const int64_t* indices,
                                    int64_t n_dst, void* dst, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0 && inner >= 1 && n_dst >= 0, "pad_by_indices: n=%lld inner=%lld n_dst=%lld", (long long)n,
                  (long long)inner, (long long)n_dst);
  ORLHF_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                  "row layout: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  if (n_dst == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(dst != nullptr && ((uintptr_t)dst & 15u) == 0, "pad_by_indices: dst must be non-NULL and 16-byte aligned");
  ORLHF_CHECK_ARG(n == 0 || (src != nullptr && indices != nullptr), "pad_by_indices: NULL argument");
  hipStream_t s = (hipStream_t)stream;
  const int64_t bytes = n_dst * inner * elem_bytes;
  hipLaunchKernelGGL(zero_bytes_kernel, dim3(flat_grid(bytes / 16 + 1)), dim3(kBlock), 0, s, (char*)dst, bytes);
  ORLHF_CHECK_LAUNCH("orlhf_pad_by_indices(zero)");
  if (n == 0) return ORLHF_OK;
  const dim3 grid(flat_grid(n * inner)), block(kBlock);
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL(scatter_index_kernel<uint8_t>, grid, block, 0, s, (const uint8_t*)src, indices, n, inner, n_dst, (uint8_t*)dst); break;
    case 2: hipLaunchKernelGGL(scatter_index_kernel<uint16_t>, grid, block, 0, s, (const uint16_t*)src, indices, n, inner, n_dst, (uint16_t*)dst); break;
    case 4: hipLaunchKernelGGL(scatter_index_kernel<uint32_t>, grid, block, 0, s, (const uint32_t*)src, indices, n, inner, n_dst, (uint32_t*)dst); break;
    default: hipLaunchKernelGGL(scatter_index_kernel<uint64_t>, grid, block, 0, s, (const uint64_t*)src, indices, n, inner, n_dst, (uint64_t*)dst); break;
  }
  ORLHF_CHECK_LAUNCH("orlhf_pad_by_indices");
  return ORLHF_OK;
}

extern "C" int orlhf_gather_by_indices(const void* src, int elem_bytes, int64_t n_src, int64_t inner, const int64_t* indices,
                                       int64_t n, void* dst, orlhf_stream_t stream) {
  ORLHF_CHECK_ARG(n >= 0 && inner >= 1 && n_src >= 0, "gather_by_indices: n=%lld inner=%lld n_src=%lld", (long long)n,
                  (long long)inner, (long long)n_src);
  ORLHF_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                  "row layout: element size %d (1, 2, 4 or 8 bytes)", elem_bytes);
  if (n == 0) return ORLHF_OK;
  ORLHF_CHECK_ARG(dst != nullptr && indices != nullptr && (src != nullptr || n_src == 0), "gather_by_indices: NULL argument");
  hipStream_t s = (hipStream_t)stream;
  const int64_t row_bytes = inner * elem_bytes;
  const uintptr_t both = (uintptr_t)src | (uintptr_t)dst | (uintptr_t)row_bytes;
  const dim3 block(kBlock);
  if ((both & 15u) == 0) {
    hipLaunchKernelGGL(gather_index_kernel<u32x4>, dim3(flat_grid(n * (row_bytes / 16))), block, 0, s, (const u32x4*)src, indices,
                       n, row_bytes / 16, n_src, (u32x4*)dst);
  } else if ((both & 7u) == 0) {
    hipLaunchKernelGGL(gather_index_kernel<uint64_t>, dim3(flat_grid(n * (row_bytes / 8))), block, 0, s, (const uint64_t*)src,
                       indices, n, row_bytes / 8, n_src, (uint64_t*)dst);
  } else if ((both & 3u) == 0) {
    hipLaunchKernelGGL(gather_index_kernel<uint32_t>, dim3(flat_grid(n * (row_bytes / 4))), block, 0, s, (const uint32_t*)src,
                       indices, n, row_bytes / 4, n_src, (uint32_t*)dst);
  } else if ((both & 1u) == 0) {
    hipLaunchKernelGGL(gather_index_kernel<uint16_t>, dim3(flat_grid(n * (row_bytes / 2))), block, 0, s, (const uint16_t*)src,
                       indices, n, row_bytes / 2, n_src, (uint16_t*)dst);
  } else {
    hipLaunchKernelGGL(gather_index_kernel<uint8_t>, dim3(flat_grid(n * row_bytes)), block, 0, s, (const uint8_t*)src, indices, n,
                       row_bytes, n_src, (uint8_t*)dst);
  }
  ORLHF_CHECK_LAUNCH("orlhf_gather_by_indices");
  return ORLHF_OK;
}
