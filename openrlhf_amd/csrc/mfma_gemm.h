// bf16 / fp16 matrix-core tile for gfx950 (CDNA4): C[256 x 256] += A[256 x K] * B[256 x K]^T with
// fp32 accumulation on v_mfma_f32_32x32x16, shared by the lm-head kernels (logits tile, and the
// two gradient products of the backward).
//
// One 256-thread workgroup (4 wave64, one per SIMD) owns a 256 x 256 output tile; wave (wm, wn)
// owns its 128 x 128 quadrant as 4 x 4 MFMA tiles of 32 x 32 (256 accumulator registers per lane).
// The K dimension is walked in slabs of 64: a slab of A and of B (32 KiB each) arrives in one LDS
// buffer while the previous slab is multiplied out of the other (two buffers of 64 KiB, one
// barrier per slab).
//
// An operand is K-major in memory (element (r, k) at r * ld + k) or MN-major (element (r, k) at
// k * ld + r). Either way its slabs go from global memory straight into LDS (buffer loads with the
// LDS bit: no registers in between), 16 bytes per lane, in the orientation they have in memory:
//   K-major slab : [256 rows][64 k], 128 B per row; 16-byte chunk kc of row r sits at position
//                  kc ^ ((r ^ (r >> 3)) & 7). A lane's MFMA fragment (one row, 8 consecutive k) is
//                  one ds_read_b128.
//   MN-major slab: [64 k][256 rows], 512 B per k; 16-byte chunk c (8 rows) of k-row k sits at
//                  position c ^ ((k & 3) << 2). A lane's fragment is two ds_read_b64_tr_b16 (the
//                  CDNA4 LDS transpose read: a group of 16 lanes reads 4 k-rows x 16 rows and
//                  every lane receives the 4 k of its own row).
// Both swizzles make the fragment reads free of bank conflicts; the LDS-direct writes are
// contiguous per instruction and cannot conflict. So the three products of the lm-head path need
// no transposed copy of any matrix and no register transposes.
//
// Bounds: a buffer resource covering the operand from the slab's first element to the end of the
// matrix makes everything past the end read as zero in hardware (no branches). For a K-major
// operand that zeroes rows past the edge; for an MN-major operand it zeroes k past the depth when
// the operand ends where its matrix ends (a sub-matrix must be multiplied with an operand that is
// zero there). Only the k tail of a K-major operand (depth not a multiple of 64) needs masking:
// that one slab goes through registers. Operand bases must be 4-byte aligned, leading dimensions
// even and below 2^23 elements (32-bit byte offsets inside a slab).
//
// MFMA 32x32x16 operand layout: lane l supplies row (l & 31), 8 consecutive k starting at
// (l >> 5) * 8; result register r of lane l is C[8 * (r / 4) + 4 * (l >> 5) + (r & 3)][l & 31].
#pragma once
#include <type_traits>
#include <utility>

#include "common.h"

namespace orlhf {
namespace mm {

constexpr int kTile = 256;            // output tile edge
constexpr int kSlab = 64;             // k elements per slab
constexpr int kThreads = 256;
constexpr int kSlabBytes = kTile * kSlab * 2;      // one operand, one slab
constexpr int kStageBytes = 2 * kSlabBytes;        // A + B
constexpr int kLdsBytes = 2 * kStageBytes;         // two stages
constexpr int64_t kMaxLd = 1ll << 23;              // leading dimensions: 255 * ld * 2 must fit 32 bits

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row ^ (row >> 3)) & 7u; }

// One operand of the product: `rows` x `depth` elements (rows = the M or N extent, depth = K).
struct Operand {
  const uint16_t* base;
  int64_t ld;      // elements between consecutive rows (K-major) or consecutive k (MN-major)
  int64_t rows;    // valid rows
  int64_t depth;   // valid k
};

// Buffer resource over the operand's memory from the element at (row0, k0) to the end of the
// matrix: loads past the end return zero in hardware. Offsets inside one slab are 32-bit; the
// 64-bit part lives in the resource's base.
template <bool MN_MAJOR>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t slab_resource(const Operand& op, int64_t row0, int64_t k0) {
  const int64_t first = MN_MAJOR ? k0 * op.ld + row0 : row0 * op.ld + k0;
  const int64_t end = MN_MAJOR ? (op.depth - 1) * op.ld + op.rows : (op.rows - 1) * op.ld + op.depth;
  int64_t bytes = ((end - first) * 2 + 3) & ~(int64_t)3;  // whole dwords: the range check is per dword
  bytes = bytes < 0 ? 0 : (bytes > 0xffffffffll ? 0xffffffffll : bytes);
  return __builtin_amdgcn_make_buffer_rsrc((void*)(op.base + first), 0, (int)(uint32_t)bytes, 0x00020000);
}

// ---- global -> LDS directly, whole slabs. One wave-instruction fills 1 KiB of LDS, lane L at byte
// 16 * L of it; a wave issues 8 of them per slab and operand. The caller waits for these loads
// (vmcnt) before the barrier that publishes the slab.
//
// K-major: instruction i of wave w covers rows (w * 8 + i) * 8 .. + 7 of the slab, lane L fetches
// the chunk that the swizzle puts at position (L & 7) of row (L >> 3) of those 8.
// MN-major: instruction i of wave w covers k-rows w * 16 + 2 i + (L >> 5), lane L fetches the chunk
// that the swizzle puts at position (L & 31) of its k-row.
template <bool MN_MAJOR>
struct SlabDma {
  __amdgpu_buffer_rsrc_t rs;
  uint32_t ld2, vbase, x, wave_u;
  char* slab;
  __device__ __forceinline__ SlabDma(const Operand& op, int64_t row0, int64_t k0, char* slab_, uint32_t wave_u_, uint32_t lane)
      : rs(slab_resource<MN_MAJOR>(op, row0, k0)), ld2((uint32_t)op.ld * 2u), wave_u(wave_u_), slab(slab_) {
    if (!MN_MAJOR) {
      const uint32_t lrow = lane >> 3;
      x = (lane & 7u) ^ lrow;  // swz(row) = (row & 7) ^ ((row >> 3) & 7) = lrow ^ i for instruction i
      vbase = lrow * ld2;
    } else {
      const uint32_t hi = lane >> 5;
      x = (lane & 31u) ^ (hi << 2);  // (k & 3) = 2 (i & 1) + hi for instruction i
      vbase = hi * ld2;
    }
  }
  __device__ __forceinline__ void issue(int i) const {
    if (!MN_MAJOR) {
      const uint32_t voff = vbase + ((x ^ (uint32_t)i) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(slab + (wave_u * 8u + i) * 1024u), 16, voff,
                                               (wave_u * 64u + (uint32_t)i * 8u) * ld2, 0, 0);
    } else {
      const uint32_t voff = vbase + ((x ^ (((uint32_t)i & 1u) << 3)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr)(slab + (wave_u * 8u + i) * 1024u), 16, voff,
                                               (wave_u * 16u + (uint32_t)i * 2u) * ld2, 0, 0);
    }
  }
};
template <bool MN_MAJOR>
__device__ __forceinline__ void dma_slab(const Operand& op, int64_t row0, int64_t k0, char* slab, uint32_t wave_u,
                                         uint32_t lane) {
  const SlabDma<MN_MAJOR> d(op, row0, k0, slab, wave_u, lane);
#pragma unroll
  for (int i = 0; i < 8; ++i) d.issue(i);
}

// ---- the k tail of a K-major operand: the slab that crosses the end of the depth goes through
// registers, where the elements past the depth (they belong to the next row) are masked out.
__device__ __forceinline__ void fetch_tail_slab(u32x4 (&r)[8], const Operand& op, int64_t row0, int64_t k0, uint32_t tid) {
  const __amdgpu_buffer_rsrc_t rs = slab_resource<false>(op, row0, k0);
  const uint32_t ld2 = (uint32_t)op.ld * 2u;
  const uint32_t kc = tid & 7u, rb = tid >> 3;
  const uint32_t voff = rb * ld2 + kc * 16u;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, (uint32_t)(32 * i) * ld2, 0);
  const int64_t valid = op.depth - (k0 + kc * 8);  // elements of this thread's chunks inside the operand
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t m = (2 * w < valid ? 0x0000ffffu : 0u) | (2 * w + 1 < valid ? 0xffff0000u : 0u);
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i][w] &= m;
  }
}
__device__ __forceinline__ void stage_tail_slab(const u32x4 (&r)[8], char* slab, uint32_t tid) {
  const uint32_t kc = tid & 7u, rb = tid >> 3;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t row = rb + 32 * i;
    *(u32x4*)(slab + row * 128u + ((kc ^ swz(row)) << 4)) = r[i];
  }
}

template <int DT>
struct Mfma;
template <>
struct Mfma<ORLHF_BF16> {
  static __device__ __forceinline__ f32x16 run(const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<ORLHF_F16> {
  static __device__ __forceinline__ f32x16 run(const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// ---- fragments of one k-step (16 k) of a slab: 4 row-tiles of A and 4 of B for this wave, each as
// two halves of 4 k (a transpose read delivers one half; the halves are joined only after the wait
// for such reads, so that no register copy can run ahead of the data)
struct Frags {
  u32x2 a[4][2], b[4][2];
};
__device__ __forceinline__ u32x4 whole(const u32x2 (&h)[2]) { return u32x4{h[0][0], h[0][1], h[1][0], h[1][1]}; }
__device__ __forceinline__ void halves(u32x2 (&h)[2], const u32x4& v) {
  h[0] = u32x2{v[0], v[1]};
  h[1] = u32x2{v[2], v[3]};
}

// The lane's coordinates in a wave's 128-row quadrant `wq` of an operand.
struct LanePos {
  uint32_t wq, lane;
};

// Row-tile t (32 rows) of k-step ks: the whole fragment of a K-major slab (one 16-byte read) ...
__device__ __forceinline__ u32x4 read_frag_k(const char* slab, int ks, int t, const LanePos& p) {  // ks, t: constants after inlining
  const uint32_t row = p.wq * 128u + (uint32_t)t * 32u + (p.lane & 31u);
  return *(const u32x4*)(slab + row * 128u + ((((uint32_t)ks * 2u + (p.lane >> 5)) ^ swz(row)) << 4));
}
// ... and half H (k 4 H .. 4 H + 3 of the lane's 8) of the fragment of an MN-major slab: lane r of a
// 16-lane group addresses k-row (r >> 2) of the group's four and rows 4 (r & 3) .. + 3 of its sixteen.
// The read is written as inline assembly: for the builtin the compiler cannot tell which LDS buffer
// is read and makes every such read wait (vmcnt(0)) for the LDS-direct loads that are in flight
// into the OTHER buffer, which serialises the whole pipeline (a third of the rate). The price is
// that the compiler does not wait for these reads either: wait_frags() below does, once per k-step.
template <int KS, int T, int H>
__device__ __forceinline__ u32x2 read_frag_mn(const char* slab, const LanePos& p) {
  const uint32_t r = p.lane & 15u, g = p.lane >> 4, q = r >> 2;
  const uint32_t k = 8u * (g >> 1) + q;                                 // + 16 KS + 4 H: in the immediate offset
  const uint32_t c = p.wq * 16u + 4u * (uint32_t)T + 2u * (g & 1u) + ((r & 3u) >> 1);
  typedef const __attribute__((address_space(3))) char* lds_bytes;
  const uint32_t at = (uint32_t)(uintptr_t)(lds_bytes)slab + k * 512u + ((c ^ (q << 2)) << 4) + (r & 1u) * 8u;
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(KS * 8192 + H * 2048));
  return v;
}
// Everything read from LDS so far has arrived; the fragments are tied to the wait, so that nothing
// that uses them is scheduled ahead of it.
__device__ __forceinline__ void wait_frags(Frags& f) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[2][0]), "+v"(f.a[2][1]),
                 "+v"(f.a[3][0]), "+v"(f.a[3][1]), "+v"(f.b[0][0]), "+v"(f.b[0][1]), "+v"(f.b[1][0]), "+v"(f.b[1][1]),
                 "+v"(f.b[2][0]), "+v"(f.b[2][1]), "+v"(f.b[3][0]), "+v"(f.b[3][1]));
}

// Read number I of a k-step's fragments, in the order a0 b0 a1 b1 ... (an MN-major operand has two
// reads per row-tile): N_READS in all.
template <bool A_MN, bool B_MN>
struct FragPlan {
  static constexpr int kA = A_MN ? 2 : 1, kB = B_MN ? 2 : 1, kPerTile = kA + kB, kReads = 4 * kPerTile;
  static constexpr bool kAsmReads = A_MN || B_MN;  // reads the compiler does not wait for: wait_frags()
  // With transpose reads in the mix all reads of a k-step go out in its first 12 slots, so that the
  // last one has four MFMAs to land before the wait at the step's end.
  static constexpr int kReadsPerSlot = kReads > 12 ? 2 : 1;
  template <int KS, int I>
  static __device__ __forceinline__ void read(Frags& f, const char* slab_a, const char* slab_b, const LanePos& pa,
                                              const LanePos& pb) {
    if constexpr (I < kReads) {
      constexpr int t = I / kPerTile, j = I % kPerTile;
      if constexpr (j < kA) {
        if constexpr (A_MN) {
          f.a[t][j] = read_frag_mn<KS, t, j>(slab_a, pa);
        } else {
          halves(f.a[t], read_frag_k(slab_a, KS, t, pa));
        }
      } else {
        constexpr int h = j - kA;
        if constexpr (B_MN) {
          f.b[t][h] = read_frag_mn<KS, t, h>(slab_b, pb);
        } else {
          halves(f.b[t], read_frag_k(slab_b, KS, t, pb));
        }
      }
    }
  }
  // the reads of pinned slot S
  template <int KS, int S>
  static __device__ __forceinline__ void read_slot(Frags& f, const char* slab_a, const char* slab_b, const LanePos& pa,
                                                   const LanePos& pb) {
    if constexpr (kReadsPerSlot == 1) {
      read<KS, S>(f, slab_a, slab_b, pa, pb);
    } else if constexpr (S < 8) {
      read<KS, 2 * S>(f, slab_a, slab_b, pa, pb);
      read<KS, 2 * S + 1>(f, slab_a, slab_b, pa, pb);
    }
  }
  template <int KS, int... I>
  static __device__ __forceinline__ void read_all(Frags& f, const char* slab_a, const char* slab_b, const LanePos& pa,
                                                  const LanePos& pb, std::integer_sequence<int, I...>) {
    (read<KS, I>(f, slab_a, slab_b, pa, pb), ...);
  }
  template <int KS>
  static __device__ __forceinline__ void read_all(Frags& f, const char* slab_a, const char* slab_b, const LanePos& pa,
                                                  const LanePos& pb) {
    read_all<KS>(f, slab_a, slab_b, pa, pb, std::make_integer_sequence<int, kReads>{});
  }
};

template <int DT>
__device__ __forceinline__ void mfma_step(f32x16 (&acc)[4][4], const Frags& f) {
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = Mfma<DT>::run(whole(f.a[mt]), whole(f.b[nt]), acc[mt][nt]);
  }
}

// One k-step with every instruction's place pinned: slot I = [LDS read I of the next fragments],
// MFMA I, [whatever `loads` issues at slot I]; nothing moves across a slot's end. Left to itself
// the scheduler issues the slab loads with their address arithmetic as one block and sinks the LDS
// reads to the end of the step, where the next step's first MFMA waits for them with the matrix
// pipe idle.
template <int DT, int I, class Reads, class Loads>
__device__ __forceinline__ void pinned_slot(f32x16 (&acc)[4][4], const Frags& use, Reads& reads, Loads& loads) {
  reads(std::integral_constant<int, I>{});
  acc[I >> 2][I & 3] = Mfma<DT>::run(whole(use.a[I >> 2]), whole(use.b[I & 3]), acc[I >> 2][I & 3]);
  loads(std::integral_constant<int, I>{});
  __builtin_amdgcn_sched_barrier(0);
}
template <int DT, class Reads, class Loads, int... I>
__device__ __forceinline__ void pinned_step(f32x16 (&acc)[4][4], const Frags& use, Reads& reads, Loads& loads,
                                            std::integer_sequence<int, I...>) {
  (pinned_slot<DT, I>(acc, use, reads, loads), ...);
}
constexpr int bits_below(uint32_t mask, int i) { return __builtin_popcount(mask & ((1u << i) - 1u)); }

// reads(S): the LDS reads of slot S for the fragments of k-step KS of a slab pair
template <bool A_MN, bool B_MN, int KS>
struct FragReads {
  Frags& f;
  const char* slab_a;
  const char* slab_b;
  const LanePos& pa;
  const LanePos& pb;
  template <int S>
  __device__ __forceinline__ void operator()(std::integral_constant<int, S>) const {
    FragPlan<A_MN, B_MN>::template read_slot<KS, S>(f, slab_a, slab_b, pa, pb);
  }
};
// loads(I): the slab pair's load number BASE + (set bits of MASK below I), if bit I of MASK is set
template <uint32_t MASK, int BASE, bool A_MN, bool B_MN>
struct SlabLoads {
  const SlabDma<A_MN>& da;
  const SlabDma<B_MN>& db;
  template <int I>
  __device__ __forceinline__ void operator()(std::integral_constant<int, I>) const {
    if constexpr (((MASK >> I) & 1u) != 0) {
      constexpr int n = BASE + bits_below(MASK, I);
      if constexpr (n < 8) da.issue(n); else db.issue(n - 8);
    }
  }
};
struct NoLoads {
  template <int I>
  __device__ __forceinline__ void operator()(std::integral_constant<int, I>) const {}
};

// Slots at which the 16 LDS-direct loads of a slab pair (8 of A, then 8 of B; per wave) are issued:
// every other slot of k-step 3 (right after the barrier that frees the buffer) and of k-step 0 of
// the next iteration, which leaves k-steps 1 and 2 for them to land. Measured against the
// alternatives at 8192^3: one load per MFMA in those two k-steps (between the LDS reads) 2-4 %
// slower; one per three MFMAs over k-steps 3, 0, 1, or any set that reaches into k-step 1, 1-4 %
// slower (the barrier then waits for the last ones); all 16 in k-step 3 3-5 % slower. Cache-policy
// bits on the loads change nothing (non-temporal: 7-20 % slower), and neither does issuing them one
// slot later in two of the four waves, so that at most two waves' loads meet at the CU's load path.
constexpr uint32_t kDmaSlots3 = 0x5555u;
constexpr uint32_t kDmaSlots0 = 0x5555u;
static_assert(__builtin_popcount(kDmaSlots3) + __builtin_popcount(kDmaSlots0) == 16, "16 loads per slab pair");

// ---- the whole product of one output tile: acc (+)= A[row0_a.., :] * B[row0_b.., :]^T over k in [0, depth)
// `lds` = kLdsBytes of dynamic shared memory. ZERO_ACC = false keeps what the caller put into acc
// (a partial sum from an earlier stretch of k: continuing it here gives the same bits as one product
// over the whole depth, since the accumulation order per element is the same).
//
// Iteration s multiplies slab s out of one LDS buffer while slab s + 1 arrives in the other: slab
// s + 2 starts towards the buffer slab s was read from as soon as the barrier of iteration s has
// freed it, a whole iteration before the barrier that publishes it, its loads on fixed slots
// between the MFMAs so that the matrix pipe never waits for a burst of address arithmetic and load
// issue. The fragments of k-step ks + 1 are read from LDS while k-step ks is multiplied; the single
// barrier of the iteration sits before the LAST k-step's MFMAs, which then cover the read of the
// next slab's first fragments: the matrix pipe does not drain at a slab boundary. Before every
// barrier that publishes a slab the wave waits for its own LDS-direct loads (s_waitcnt vmcnt(0):
// the compiler's bookkeeping of these loads is not relied on).
// RESIDENT_OPERANDS (measurement only): the steady loop issues no slab loads, every slab is
// multiplied out of whatever the LDS buffers hold. The result is meaningless; the time is what the
// same LDS reads, MFMAs and barriers take when nothing else uses the LDS and the load path.
template <int DT, bool A_MN, bool B_MN, bool ZERO_ACC = true, bool RESIDENT_OPERANDS = false>
__device__ __forceinline__ void tile_product(f32x16 (&acc)[4][4], const Operand& a, const Operand& b, int64_t row0_a,
                                             int64_t row0_b, char* lds) {
  // Everything addressed below derives from the thread index: making it opaque keeps a caller's
  // loop over tiles from hoisting a hundred address registers out of the product and holding
  // them (spilled) across its epilogue; they are recomputed per tile instead.
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
  const LanePos pa{wave & 1u, lane}, pb{wave >> 1, lane};
  using Plan = FragPlan<A_MN, B_MN>;
  if (ZERO_ACC) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;
      }
    }
  }
  const int64_t depth = a.depth;
  const int64_t n_slabs = (depth + kSlab - 1) / kSlab;
  // slabs 0 .. n_dma - 1 go straight into LDS; a last slab that crosses the end of the depth needs
  // masking if an operand is K-major
  const int64_t n_dma = (A_MN && B_MN) ? n_slabs : depth / kSlab;
  // slab `sl` of both operands into the buffer at `stage`; the caller waits (vmcnt) and synchronises
  auto load_slab = [&](int64_t sl, char* stage) {
    if (A_MN || sl < n_dma) {
      dma_slab<A_MN>(a, row0_a, sl * kSlab, stage, wave_u, lane);
    } else {
      u32x4 r[8];
      fetch_tail_slab(r, a, row0_a, sl * kSlab, tid);
      stage_tail_slab(r, stage, tid);
      __builtin_amdgcn_sched_barrier(0);  // A's registers are free again before B's are loaded
    }
    if (B_MN || sl < n_dma) {
      dma_slab<B_MN>(b, row0_b, sl * kSlab, stage + kSlabBytes, wave_u, lane);
    } else {
      u32x4 r[8];
      fetch_tail_slab(r, b, row0_b, sl * kSlab, tid);
      stage_tail_slab(r, stage + kSlabBytes, tid);
    }
  };
  load_slab(0, lds);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  constexpr int n3 = __builtin_popcount(kDmaSlots3);
  using Slots16 = std::make_integer_sequence<int, 16>;
  if (n_dma > 1 && !RESIDENT_OPERANDS) {  // slab 1 is whole: its first loads start towards the second buffer now
    const SlabDma<A_MN> da(a, row0_a, kSlab, lds + kStageBytes, wave_u, lane);
    const SlabDma<B_MN> db(b, row0_b, kSlab, lds + kStageBytes + kSlabBytes, wave_u, lane);
#pragma unroll
    for (int n = 0; n < n3; ++n) {
      if (n < 8) da.issue(n); else db.issue(n - 8);
    }
  }
  Frags f0, f1;
  Plan::template read_all<0>(f0, lds, lds + kSlabBytes, pa, pb);
  int64_t s = 0;

  // One steady-state iteration: slab `it` in buffer PARITY; slab it + 1 (whole) has had its first
  // loads since k-step 3 of the previous iteration and gets the rest in k-step 0; after the barrier
  // slab it + 2 starts towards `cur` (in the last iteration slab 0 again instead of a branch:
  // nobody reads it, and whatever touches this buffer next waits for its own later loads, which
  // complete after these).
  auto steady = [&](auto parity, int64_t it) {
    constexpr int P = decltype(parity)::value;
    char* cur = lds + P * kStageBytes;
    char* nxt = lds + (1 - P) * kStageBytes;
    const int64_t k1 = (it + 1) * kSlab, k2 = it + 2 < n_dma ? (it + 2) * kSlab : 0;
    const SlabDma<A_MN> da1(a, row0_a, k1, nxt, wave_u, lane);
    const SlabDma<B_MN> db1(b, row0_b, k1, nxt + kSlabBytes, wave_u, lane);
    NoLoads none;
    {
      FragReads<A_MN, B_MN, 1> rd{f1, cur, cur + kSlabBytes, pa, pb};
      SlabLoads<kDmaSlots0, n3, A_MN, B_MN> ld{da1, db1};
      if (Plan::kAsmReads) wait_frags(f0);
      if (RESIDENT_OPERANDS) pinned_step<DT>(acc, f0, rd, none, Slots16{}); else pinned_step<DT>(acc, f0, rd, ld, Slots16{});
    }
    {
      FragReads<A_MN, B_MN, 2> rd{f0, cur, cur + kSlabBytes, pa, pb};
      if (Plan::kAsmReads) wait_frags(f1);
      pinned_step<DT>(acc, f1, rd, none, Slots16{});
    }
    {
      FragReads<A_MN, B_MN, 3> rd{f1, cur, cur + kSlabBytes, pa, pb};
      if (Plan::kAsmReads) wait_frags(f0);
      pinned_step<DT>(acc, f0, rd, none, Slots16{});
    }
    // every wave holds its last fragments of `cur`; slab it + 1 is complete in `nxt`
    if (Plan::kAsmReads) wait_frags(f1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const SlabDma<A_MN> da2(a, row0_a, k2, cur, wave_u, lane);
    const SlabDma<B_MN> db2(b, row0_b, k2, cur + kSlabBytes, wave_u, lane);
    {
      FragReads<A_MN, B_MN, 0> rd{f0, nxt, nxt + kSlabBytes, pa, pb};
      SlabLoads<kDmaSlots3, 0, A_MN, B_MN> ld{da2, db2};
      if (RESIDENT_OPERANDS) pinned_step<DT>(acc, f1, rd, none, Slots16{}); else pinned_step<DT>(acc, f1, rd, ld, Slots16{});
    }
  };
  for (; s + 2 < n_dma; s += 2) {  // pairs of steady iterations: the buffers' addresses are constants
    steady(std::integral_constant<int, 0>{}, s);
    steady(std::integral_constant<int, 1>{}, s + 1);
  }
  if (s + 1 < n_dma) {  // s is even here
    steady(std::integral_constant<int, 0>{}, s);
    ++s;
  }
  // s == max(n_dma - 1, 0): slab s is in its buffer and f0 holds its first fragments; what is left
  // is that slab and, after it, the one that crosses the end of the depth (if there is one)
  for (; s < n_slabs; ++s) {
    const char* cur = lds + (s & 1) * kStageBytes;
    char* nxt = lds + ((s + 1) & 1) * kStageBytes;
    const bool has1 = s + 1 < n_slabs;
    if (Plan::kAsmReads) wait_frags(f0);
    Plan::template read_all<1>(f1, cur, cur + kSlabBytes, pa, pb);
    mfma_step<DT>(acc, f0);
    if (Plan::kAsmReads) wait_frags(f1);
    Plan::template read_all<2>(f0, cur, cur + kSlabBytes, pa, pb);
    mfma_step<DT>(acc, f1);
    if (Plan::kAsmReads) wait_frags(f0);
    Plan::template read_all<3>(f1, cur, cur + kSlabBytes, pa, pb);
    mfma_step<DT>(acc, f0);
    if (Plan::kAsmReads) wait_frags(f1);
    if (has1) {
      // `nxt` was last read in iteration s - 1, whose barrier every wave has passed; the loads
      // below are younger than any load still on its way there and complete after it
      load_slab(s + 1, nxt);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      Plan::template read_all<0>(f0, nxt, nxt + kSlabBytes, pa, pb);
    }
    mfma_step<DT>(acc, f1);
  }
  // the reload that stood in for a missing slab may still be on its way into LDS: it is long
  // done by now, the wait only makes that explicit for whoever touches the buffers next
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // no closing barrier: after the barrier inside the last iteration no wave reads the slab
  // buffers any more, but a caller that reuses them as scratch must synchronise first
}

// Position of accumulator register r of tile (mt, nt) inside the 256 x 256 output tile.
__device__ __forceinline__ uint32_t acc_row(uint32_t wm, int mt, int r, uint32_t lane) {
  return wm * 128u + mt * 32u + 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3);
}
__device__ __forceinline__ uint32_t acc_col(uint32_t wn, int nt, uint32_t lane) { return wn * 128u + nt * 32u + (lane & 31u); }

// Workgroup index -> tile index such that the workgroups of one XCD (indices congruent modulo 8)
// work on a contiguous range of tiles and share operand rows through that XCD's L2.
__device__ __forceinline__ uint32_t xcd_contiguous(uint32_t wg, uint32_t n) {
  const uint32_t per = (n + 7u) / 8u;
  return (wg & 7u) * per + (wg >> 3);  // may be >= n for the last XCD's slack: callers skip those
}

// Work item t of a tiles_m x tiles_n grid -> (tm, tn) such that 32 consecutive items (what one
// XCD runs at a time) form an 8 x 4 block: 12 distinct operand row-blocks for 32 tiles, so most
// slab loads hit that XCD's L2. (Tile counts are below 2^31: checked by the host.)
__device__ __forceinline__ void grouped_tile(uint32_t t, uint32_t tiles_m, uint32_t tiles_n, uint32_t& tm, uint32_t& tn) {
  const uint32_t per_group = 8u * tiles_n;
  const uint32_t group = t / per_group, in_group = t - group * per_group;
  const uint32_t first = group * 8u;
  const uint32_t height = tiles_m - first < 8u ? tiles_m - first : 8u;
  tn = in_group / height;
  tm = first + (in_group - tn * height);
}

}  // namespace mm
}  // namespace orlhf
