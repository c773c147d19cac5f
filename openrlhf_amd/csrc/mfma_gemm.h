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
// LDS layout of a slab: [256 rows][64 k] 16-bit elements, i.e. 8 chunks of 16 bytes per row; chunk
// kc of row r sits at position kc ^ swz(r), swz(r) = (r ^ (r >> 3)) & 7, which makes the staging
// writes and the fragment reads (32 consecutive rows, one chunk each) conflict-free.
//
// Global loads are buffer loads: a resource covering the operand from the slab's first element to
// the end of the matrix makes rows past the edge read as zero in hardware (no branches); only a k
// tail of a K-major operand (depth not a multiple of 64) is masked in registers, in a separate
// copy of the loop that runs for the last slab alone. Operand bases must be 4-byte aligned and
// leading dimensions even.
//
// An operand may be K-major in memory (element (r, k) at r * ld + k: copied chunk by chunk) or
// MN-major (element (r, k) at k * ld + r: each thread fetches an 8 x 8 block, transposes it in
// registers with byte permutes and writes 8 chunks), so the three products of the lm-head path
// need no transposed copy of any matrix.
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

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(2)));  // 16 bytes at element alignment

__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row ^ (row >> 3)) & 7u; }

// One operand of the product: `rows` x `depth` elements (rows = the M or N extent, depth = K).
struct Operand {
  const uint16_t* base;
  int64_t ld;      // elements between consecutive rows (K-major) or consecutive k (MN-major)
  int64_t rows;    // valid rows; rows beyond read as zero
  int64_t depth;   // valid k; k beyond reads as zero
};

// Buffer resource over the operand's memory from the element at (row0, k0) to the end of the
// matrix: loads past the end return zero in hardware, so rows beyond the operand need no branch.
// Offsets inside one slab are 32-bit; the 64-bit part lives in the resource's base.
template <bool MN_MAJOR>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t slab_resource(const Operand& op, int64_t row0, int64_t k0) {
  const int64_t first = MN_MAJOR ? k0 * op.ld + row0 : row0 * op.ld + k0;
  const int64_t end = MN_MAJOR ? (op.depth - 1) * op.ld + op.rows : (op.rows - 1) * op.ld + op.depth;
  int64_t bytes = ((end - first) * 2 + 3) & ~(int64_t)3;  // whole dwords: the range check is per dword
  bytes = bytes < 0 ? 0 : (bytes > 0xffffffffll ? 0xffffffffll : bytes);
  return __builtin_amdgcn_make_buffer_rsrc((void*)(op.base + first), 0, (int)(uint32_t)bytes, 0x00020000);
}

// ---- global -> registers: the 8 chunks of one thread for the slab starting at k0, rows row0..
// Rows beyond the operand read as zero (K-major) or as whatever follows (MN-major, where they
// only reach output rows nobody stores); k beyond the operand must read as zero for both, which
// the resource does for MN-major and TAIL masks in registers for K-major (the elements past
// `depth` in a row belong to the next row).
template <bool MN_MAJOR, bool TAIL, int I0 = 0, int I1 = 8>
__device__ __forceinline__ void fetch_slab(u32x4 (&r)[8], const Operand& op, int64_t row0, int64_t k0, uint32_t tid) {
  const __amdgpu_buffer_rsrc_t rs = slab_resource<MN_MAJOR>(op, row0, k0);
  const uint32_t ld2 = (uint32_t)op.ld * 2u;
  if (!MN_MAJOR) {
    const uint32_t kc = tid & 7u, rb = tid >> 3;
    const uint32_t voff = rb * ld2 + kc * 16u;
#pragma unroll
    for (int i = I0; i < I1; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, (uint32_t)(32 * i) * ld2, 0);
    if (TAIL) {
      const int64_t valid = op.depth - (k0 + kc * 8);  // elements of this thread's chunks inside the operand
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t m = (2 * w < valid ? 0x0000ffffu : 0u) | (2 * w + 1 < valid ? 0xffff0000u : 0u);
#pragma unroll
        for (int i = I0; i < I1; ++i) r[i][w] &= m;
      }
    }
  } else {
    const uint32_t c = tid & 31u, kb = tid >> 5;
    const uint32_t voff = kb * 8u * ld2 + c * 16u;
#pragma unroll
    for (int i = I0; i < I1; ++i) r[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, (uint32_t)i * ld2, 0);
  }
}

// ---- global -> LDS directly (K-major operands, whole slabs): buffer loads that write LDS without
// passing through registers. One wave-instruction fills 1 KiB of LDS, lane L at byte 16 * L: 8 rows
// of the slab, so lane L fetches the chunk that the swizzle puts at position (L & 7) of row
// (L >> 3) of those 8 rows. Rows past the operand arrive as zeros (resource bounds). The caller
// waits for these loads (vmcnt) before the barrier that publishes the slab.
struct SlabDma {
  __amdgpu_buffer_rsrc_t rs;
  uint32_t ld2, vbase, x, wave_u;
  char* slab;
  __device__ __forceinline__ SlabDma(const Operand& op, int64_t row0, int64_t k0, char* slab_, uint32_t wave_u_, uint32_t lane)
      : rs(slab_resource<false>(op, row0, k0)), ld2((uint32_t)op.ld * 2u), wave_u(wave_u_), slab(slab_) {
    const uint32_t lrow = lane >> 3;
    x = (lane & 7u) ^ lrow;
    vbase = lrow * ld2;
  }
  // load i of this wave's 8: rows (wave_u * 8 + i) * 8 .. + 7, swz(row) = (row & 7) ^ ((row >> 3) & 7) = lrow ^ i
  __device__ __forceinline__ void issue(int i) const {
    const uint32_t voff = vbase + ((x ^ (uint32_t)i) << 4);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(slab + (wave_u * 8u + i) * 1024u), 16,
                                             voff, (wave_u * 64u + (uint32_t)i * 8u) * ld2, 0, 0);
  }
};
__device__ __forceinline__ void dma_slab(const Operand& op, int64_t row0, int64_t k0, char* slab, uint32_t wave_u,
                                         uint32_t lane) {
  const SlabDma d(op, row0, k0, slab, wave_u, lane);
#pragma unroll
  for (int i = 0; i < 8; ++i) d.issue(i);
}

// ---- registers -> LDS slab ([256][64] swizzled). K-major: chunks I0 .. I1-1 of this thread.
// MN-major: the 8 x 8 block is transposed as a whole; output rows E0 .. E1-1 are written.
template <bool MN_MAJOR, int I0 = 0, int I1 = 8>
__device__ __forceinline__ void stage_slab(const u32x4 (&r)[8], char* slab, uint32_t tid) {
  if (!MN_MAJOR) {
    const uint32_t kc = tid & 7u, rb = tid >> 3;
#pragma unroll
    for (int i = I0; i < I1; ++i) {
      const uint32_t row = rb + 32 * i;
      *(u32x4*)(slab + row * 128u + ((kc ^ swz(row)) << 4)) = r[i];
    }
  } else {
    // r[i] = 8 consecutive rows at k = 8*kb + i  ->  t[e] = 8 consecutive k of row 8*c + e
    const uint32_t c = tid & 31u, kb = tid >> 5;
#pragma unroll
    for (int e = I0; e < I1; ++e) {
      u32x4 t;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = r[2 * j][e >> 1], hi = r[2 * j + 1][e >> 1];
        t[j] = (e & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
      }
      const uint32_t row = c * 8 + e;
      *(u32x4*)(slab + row * 128u + ((kb ^ swz(row)) << 4)) = t;
    }
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

// ---- fragments of one k-step (16 k) of a slab: 4 row-tiles of A and 4 of B for this wave
struct Frags {
  u32x4 a[4], b[4];
};

__device__ __forceinline__ void load_frags(Frags& f, const char* slab_a, const char* slab_b, int ks, uint32_t wm,
                                           uint32_t wn, uint32_t lane) {
  const uint32_t lr = lane & 31u, lk = lane >> 5;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const uint32_t ra = wm * 128u + t * 32u + lr, rb = wn * 128u + t * 32u + lr;
    f.a[t] = *(const u32x4*)(slab_a + ra * 128u + (((ks * 2u + lk) ^ swz(ra)) << 4));
    f.b[t] = *(const u32x4*)(slab_b + rb * 128u + (((ks * 2u + lk) ^ swz(rb)) << 4));
  }
}

template <int DT>
__device__ __forceinline__ void mfma_step(f32x16 (&acc)[4][4], const Frags& f) {
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = Mfma<DT>::run(f.a[mt], f.b[nt], acc[mt][nt]);
  }
}

// Issue order of one k-step of the steady loop: the eight LDS reads of the next fragments, and
// N_VMEM global loads into registers per read, go out under the first eight MFMAs; the other eight
// MFMAs cover their latency. Left to itself the scheduler sinks the reads to the end of the step,
// where the next step's first MFMA waits for them with the matrix pipe idle. (Used by the
// iteration with two register operands only; the others pin every slot.)
template <int N_VMEM>
__device__ __forceinline__ void issue_order() {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
    if (N_VMEM > 0) __builtin_amdgcn_sched_group_barrier(0x010, N_VMEM, 0);  // global loads into registers
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
}

// Before the barrier that publishes a slab, its LDS-direct loads must have landed. The compiler's
// own bookkeeping of these loads is not relied on (it left the wait out at one of the two barriers
// of an unrolled iteration pair): loads retire in order, so allowing the YOUNGER loads that were
// issued since (the 8 register loads of an operand carried in registers) to be outstanding waits
// exactly for the slab.
template <int YOUNGER>
__device__ __forceinline__ void wait_slab_loads() {
  static_assert(YOUNGER == 0 || YOUNGER == 8 || YOUNGER == 16, "8 register loads per operand and slab");
  if (YOUNGER == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (YOUNGER == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
}

// One k-step with every instruction's place pinned: slot I = [LDS read I of the next fragments (I < 8)],
// MFMA I, [whatever `loads` issues at slot I]; nothing moves across a slot's end.
template <int DT, int I, class Reads, class Loads>
__device__ __forceinline__ void pinned_slot(f32x16 (&acc)[4][4], const Frags& use, Reads& reads, Loads& loads) {
  reads(std::integral_constant<int, I>{});
  acc[I >> 2][I & 3] = Mfma<DT>::run(use.a[I >> 2], use.b[I & 3], acc[I >> 2][I & 3]);
  loads(std::integral_constant<int, I>{});
  __builtin_amdgcn_sched_barrier(0);
}
template <int DT, class Reads, class Loads, int... I>
__device__ __forceinline__ void pinned_step(f32x16 (&acc)[4][4], const Frags& use, Reads& reads, Loads& loads,
                                            std::integer_sequence<int, I...>) {
  (pinned_slot<DT, I>(acc, use, reads, loads), ...);
}
constexpr int bits_below(uint32_t mask, int i) { return __builtin_popcount(mask & ((1u << i) - 1u)); }

// reads(I): LDS read I (a0 b0 a1 b1 ...) of the fragments of k-step `ks2 / 2` of a slab
struct FragReads {
  Frags& f;
  const char* slab_a;
  const char* slab_b;
  uint32_t ks2, wm, wn, lr, lk;
  template <int I>
  __device__ __forceinline__ void operator()(std::integral_constant<int, I>) const {
    if constexpr (I < 8) {
      constexpr int t = I >> 1;
      if constexpr ((I & 1) == 0) {
        const uint32_t ra = wm * 128u + t * 32u + lr;
        f.a[t] = *(const u32x4*)(slab_a + ra * 128u + (((ks2 + lk) ^ swz(ra)) << 4));
      } else {
        const uint32_t rb = wn * 128u + t * 32u + lr;
        f.b[t] = *(const u32x4*)(slab_b + rb * 128u + (((ks2 + lk) ^ swz(rb)) << 4));
      }
    }
  }
};
// loads(I): the slab pair's load number BASE + (set bits of MASK below I), if bit I of MASK is set
template <uint32_t MASK, int BASE>
struct SlabLoads {
  const SlabDma& da;
  const SlabDma& db;
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
constexpr uint32_t kDmaSlots1 = 0x0u;
static_assert(__builtin_popcount(kDmaSlots3) + __builtin_popcount(kDmaSlots0) + __builtin_popcount(kDmaSlots1) == 16, "16 loads per slab pair");

// ---- the whole product of one output tile: acc = A[row0_a.., :] * B[row0_b.., :]^T over k in [0, depth)
// `lds` = kLdsBytes of dynamic shared memory.
//
// Iteration s multiplies slab s out of one LDS buffer while slab s + 1 is (or arrives) in the other:
//  * a K-major operand's slab is loaded straight into LDS (SlabDma): slab s + 2 as soon as the
//    barrier of iteration s has freed the buffer slab s was read from, a whole iteration before
//    the barrier that publishes it, its loads on fixed slots between the MFMAs (steady_kk,
//    steady_mixed below) so that the matrix pipe never waits for a burst of address arithmetic
//    and load issue; only a slab that crosses the end of the depth goes through registers (masking);
//  * an MN-major operand's slab s + 1 sits in registers (fetched during iteration s - 1), is
//    transposed and written to LDS during the first k-steps, and the fetch of slab s + 2 is issued
//    into the registers it leaves.
// The fragments of k-step ks + 1 are read from LDS while k-step ks is multiplied; the single
// barrier of the iteration sits before the LAST k-step's MFMAs, which then cover the read of the
// next slab's first fragments: the matrix pipe does not drain at a slab boundary.
// (Touching slab s + 2 an iteration early to warm the L2 changed nothing: the counters put the
// average L2 read latency of these loads at ~270 cycles, far below an iteration.)
// RESIDENT_OPERANDS (measurement only): the steady loop issues no slab loads, every slab is
// multiplied out of whatever the LDS buffers hold. The result is meaningless; the time is what the
// same LDS reads, MFMAs and barriers take when nothing else uses the LDS and the load path.
template <int DT, bool A_MN_MAJOR, bool B_MN_MAJOR, bool RESIDENT_OPERANDS = false>
__device__ __forceinline__ void tile_product(f32x16 (&acc)[4][4], const Operand& a, const Operand& b, int64_t row0_a,
                                             int64_t row0_b, char* lds) {
  // Everything addressed below derives from the thread index: making it opaque keeps a caller's
  // loop over tiles from hoisting a hundred address registers out of the product and holding
  // them (spilled) across its epilogue; they are recomputed per tile instead.
  // operands whose next slab is carried in registers (K-major ones through registers as well were
  // 3-11 % slower than the LDS-direct loads)
  constexpr bool A_REG = A_MN_MAJOR, B_REG = B_MN_MAJOR;
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t wm = wave & 1u, wn = wave >> 1;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;
    }
  }
  const int64_t depth = a.depth;
  const int64_t n_slabs = (depth + kSlab - 1) / kSlab;
  const int64_t full = depth / kSlab;  // slabs 0 .. full-1 are whole
  u32x4 ra[8], rb[8];
  fetch_slab<A_MN_MAJOR, true>(ra, a, row0_a, 0, tid);
  fetch_slab<B_MN_MAJOR, true>(rb, b, row0_b, 0, tid);
  stage_slab<A_MN_MAJOR>(ra, lds, tid);
  stage_slab<B_MN_MAJOR>(rb, lds + kSlabBytes, tid);
  if (n_slabs > 1) {  // MN-major operands carry slab s + 1 in registers from one iteration to the next
    if (A_REG) fetch_slab<A_MN_MAJOR, true>(ra, a, row0_a, kSlab, tid);
    if (B_REG) fetch_slab<B_MN_MAJOR, true>(rb, b, row0_b, kSlab, tid);
  }
  __syncthreads();
  constexpr bool KK = !A_REG && !B_REG;  // both slabs by LDS-direct loads: the pinned schedule
  constexpr int n3 = __builtin_popcount(kDmaSlots3), n0 = __builtin_popcount(kDmaSlots0);
  using Slots16 = std::make_integer_sequence<int, 16>;
  if (full > 1) {  // slab 1 is whole: its first loads start towards the second buffer now
    if (KK) {
      if (!RESIDENT_OPERANDS) {
        const SlabDma da(a, row0_a, kSlab, lds + kStageBytes, wave_u, lane);
        const SlabDma db(b, row0_b, kSlab, lds + kStageBytes + kSlabBytes, wave_u, lane);
#pragma unroll
        for (int n = 0; n < n3; ++n) {
          if (n < 8) da.issue(n); else db.issue(n - 8);
        }
      }
    } else if (!A_REG) {
      dma_slab(a, row0_a, kSlab, lds + kStageBytes, wave_u, lane);
    }
  }
  Frags f0, f1;
  load_frags(f0, lds, lds + kSlabBytes, 0, wm, wn, lane);
  int64_t s = 0;

  // One steady-state iteration: slab `it` in buffer PARITY; slab it + 1 is whole and lands in (or
  // is staged into) the other buffer. Needs it + 1 < full. This version is for two operands
  // carried in registers (no caller of the library has two MN-major operands): the issue order
  // is left to the scheduler groups of issue_order.
  auto steady = [&](auto parity, int64_t it) {
    constexpr int P = decltype(parity)::value;
    char* cur = lds + P * kStageBytes;
    char* nxt = lds + (1 - P) * kStageBytes;
    const int64_t k2 = (it + 2) * kSlab;
    // k-step 0
    load_frags(f1, cur, cur + kSlabBytes, 1, wm, wn, lane);
    stage_slab<A_MN_MAJOR, 0, 4>(ra, nxt, tid);
    stage_slab<B_MN_MAJOR, 0, 4>(rb, nxt + kSlabBytes, tid);
    mfma_step<DT>(acc, f0);
    issue_order<0>();
    __builtin_amdgcn_sched_barrier(0);
    // k-step 1
    load_frags(f0, cur, cur + kSlabBytes, 2, wm, wn, lane);
    stage_slab<A_MN_MAJOR, 4, 8>(ra, nxt, tid);
    stage_slab<B_MN_MAJOR, 4, 8>(rb, nxt + kSlabBytes, tid);
    mfma_step<DT>(acc, f1);
    issue_order<0>();
    __builtin_amdgcn_sched_barrier(0);
    // k-step 2
    load_frags(f1, cur, cur + kSlabBytes, 3, wm, wn, lane);
    fetch_slab<A_MN_MAJOR, !A_MN_MAJOR>(ra, a, row0_a, k2, tid);
    fetch_slab<B_MN_MAJOR, !B_MN_MAJOR>(rb, b, row0_b, k2, tid);
    mfma_step<DT>(acc, f0);
    issue_order<2>();
    // every wave holds its last fragments of `cur`; slab it + 1 is complete in `nxt`
    __syncthreads();
    // k-step 3, over the read of the next slab's first fragments
    load_frags(f0, nxt, nxt + kSlabBytes, 0, wm, wn, lane);
    mfma_step<DT>(acc, f1);
    issue_order<0>();
    __builtin_amdgcn_sched_barrier(0);
  };
  // The same iteration when both operands arrive by LDS-direct loads: slab it + 1 has had its first
  // loads since k-step 3 of the previous iteration and gets the rest in k-steps 0 and 1; after the
  // barrier slab it + 2 starts towards `cur` (in the last iteration slab 0 again instead of a branch:
  // nobody reads it, and whatever touches this buffer next waits for its own later loads).
  auto steady_kk = [&](auto parity, int64_t it) {
    constexpr int P = decltype(parity)::value;
    char* cur = lds + P * kStageBytes;
    char* nxt = lds + (1 - P) * kStageBytes;
    const int64_t k1 = (it + 1) * kSlab, k2 = it + 2 < full ? (it + 2) * kSlab : 0;
    const uint32_t lr = lane & 31u, lk = lane >> 5;
    const SlabDma da1(a, row0_a, k1, nxt, wave_u, lane), db1(b, row0_b, k1, nxt + kSlabBytes, wave_u, lane);
    NoLoads none;
    {
      FragReads rd{f1, cur, cur + kSlabBytes, 2, wm, wn, lr, lk};
      SlabLoads<kDmaSlots0, n3> ld{da1, db1};
      if (RESIDENT_OPERANDS) pinned_step<DT>(acc, f0, rd, none, Slots16{}); else pinned_step<DT>(acc, f0, rd, ld, Slots16{});
    }
    {
      FragReads rd{f0, cur, cur + kSlabBytes, 4, wm, wn, lr, lk};
      SlabLoads<kDmaSlots1, n3 + n0> ld{da1, db1};
      if (RESIDENT_OPERANDS) pinned_step<DT>(acc, f1, rd, none, Slots16{}); else pinned_step<DT>(acc, f1, rd, ld, Slots16{});
    }
    {
      FragReads rd{f1, cur, cur + kSlabBytes, 6, wm, wn, lr, lk};
      pinned_step<DT>(acc, f0, rd, none, Slots16{});
    }
    // every wave holds its last fragments of `cur`; slab it + 1 is complete in `nxt`
    wait_slab_loads<0>();
    __syncthreads();
    const SlabDma da2(a, row0_a, k2, cur, wave_u, lane), db2(b, row0_b, k2, cur + kSlabBytes, wave_u, lane);
    {
      FragReads rd{f0, nxt, nxt + kSlabBytes, 0, wm, wn, lr, lk};
      SlabLoads<kDmaSlots3, 0> ld{da2, db2};
      if (RESIDENT_OPERANDS) pinned_step<DT>(acc, f1, rd, none, Slots16{}); else pinned_step<DT>(acc, f1, rd, ld, Slots16{});
    }
  };
  // The same iteration with one operand carried in registers, every instruction in a fixed slot:
  // the register operand's slab it + 1 is written to LDS on the odd slots behind the LDS reads of
  // k-steps 0 and 1 (four rows each), its slab it + 2 is fetched on the odd slots of k-step 2;
  // the other operand's LDS-direct loads take the even slots of k-step 0 (B) or k-step 3 (A).
  auto steady_mixed = [&](auto parity, int64_t it) {
    constexpr int P = decltype(parity)::value;
    char* cur = lds + P * kStageBytes;
    char* nxt = lds + (1 - P) * kStageBytes;
    const int64_t k1 = (it + 1) * kSlab, k2 = (it + 2) * kSlab;
    const uint32_t lr = lane & 31u, lk = lane >> 5;
    const SlabDma db(b, row0_b, k1, nxt + kSlabBytes, wave_u, lane);  // B's slab it + 1 (unused if B_REG)
    auto stage_rows = [&](auto first) {  // rows FIRST .. FIRST + 3 on slots 9, 11, 13, 15
      return [&, first](auto ic) {
        constexpr int I = decltype(ic)::value, F = decltype(first)::value;
        if constexpr (I >= 9 && (I & 1) == 1) {
          constexpr int e = F + (I - 9) / 2;
          if (A_REG) stage_slab<A_MN_MAJOR, e, e + 1>(ra, nxt, tid);
          if (B_REG) stage_slab<B_MN_MAJOR, e, e + 1>(rb, nxt + kSlabBytes, tid);
        }
      };
    };
    {
      FragReads rd{f1, cur, cur + kSlabBytes, 2, wm, wn, lr, lk};
      auto stage = stage_rows(std::integral_constant<int, 0>{});
      auto extra = [&](auto ic) {
        constexpr int I = decltype(ic)::value;
        if constexpr (!B_REG && (I & 1) == 0) db.issue(I / 2);
        stage(ic);
      };
      pinned_step<DT>(acc, f0, rd, extra, Slots16{});
    }
    {
      FragReads rd{f0, cur, cur + kSlabBytes, 4, wm, wn, lr, lk};
      auto stage = stage_rows(std::integral_constant<int, 4>{});
      pinned_step<DT>(acc, f1, rd, stage, Slots16{});
    }
    {
      FragReads rd{f1, cur, cur + kSlabBytes, 6, wm, wn, lr, lk};
      auto fetch = [&](auto ic) {
        constexpr int I = decltype(ic)::value;
        if constexpr ((I & 1) == 1) {
          constexpr int i = I / 2;
          if (A_REG) fetch_slab<A_MN_MAJOR, !A_MN_MAJOR, i, i + 1>(ra, a, row0_a, k2, tid);
          if (B_REG) fetch_slab<B_MN_MAJOR, !B_MN_MAJOR, i, i + 1>(rb, b, row0_b, k2, tid);
        }
      };
      pinned_step<DT>(acc, f0, rd, fetch, Slots16{});
    }
    // every wave holds its last fragments of `cur`; slab it + 1 is complete in `nxt`
    wait_slab_loads<8>();
    __syncthreads();
    const SlabDma da(a, row0_a, it + 2 < full ? k2 : 0, cur, wave_u, lane);  // A's slab it + 2 (unused if A_REG)
    {
      FragReads rd{f0, nxt, nxt + kSlabBytes, 0, wm, wn, lr, lk};
      auto extra = [&](auto ic) {
        constexpr int I = decltype(ic)::value;
        if constexpr (!A_REG && (I & 1) == 0) da.issue(I / 2);
      };
      pinned_step<DT>(acc, f1, rd, extra, Slots16{});
    }
  };
  auto iteration = [&](auto parity, int64_t it) {
    if constexpr (KK) steady_kk(parity, it);
    else if constexpr (A_REG != B_REG) steady_mixed(parity, it);
    else steady(parity, it);
  };
  for (; s + 2 < full; s += 2) {  // pairs of steady iterations: the buffers' addresses are constants
    iteration(std::integral_constant<int, 0>{}, s);
    iteration(std::integral_constant<int, 1>{}, s + 1);
  }
  if (s + 1 < full) {  // s is even here
    iteration(std::integral_constant<int, 0>{}, s);
    ++s;
  }
  // s == full - 1 (or 0): slab s is in its buffer, no load into LDS is outstanding
  for (; s < n_slabs; ++s) {  // the last slabs: a k tail may need masking, slabs run out
    const char* cur = lds + (s & 1) * kStageBytes;
    char* nxt = lds + ((s + 1) & 1) * kStageBytes;
    const bool has1 = s + 1 < n_slabs, has2 = s + 2 < n_slabs;
    if (has1) {
      if (!A_REG) fetch_slab<false, true>(ra, a, row0_a, (s + 1) * kSlab, tid);
      if (!B_REG) fetch_slab<false, true>(rb, b, row0_b, (s + 1) * kSlab, tid);
      if (A_REG) stage_slab<A_MN_MAJOR>(ra, nxt, tid);
      if (B_REG) stage_slab<B_MN_MAJOR>(rb, nxt + kSlabBytes, tid);
    }
    if (has2) {
      if (A_REG) fetch_slab<A_MN_MAJOR, true>(ra, a, row0_a, (s + 2) * kSlab, tid);
      if (B_REG) fetch_slab<B_MN_MAJOR, true>(rb, b, row0_b, (s + 2) * kSlab, tid);
    }
    load_frags(f1, cur, cur + kSlabBytes, 1, wm, wn, lane);
    mfma_step<DT>(acc, f0);
    load_frags(f0, cur, cur + kSlabBytes, 2, wm, wn, lane);
    mfma_step<DT>(acc, f1);
    load_frags(f1, cur, cur + kSlabBytes, 3, wm, wn, lane);
    mfma_step<DT>(acc, f0);
    if (has1) {
      if (!A_REG) stage_slab<false>(ra, nxt, tid);
      if (!B_REG) stage_slab<false>(rb, nxt + kSlabBytes, tid);
      __syncthreads();
      load_frags(f0, nxt, nxt + kSlabBytes, 0, wm, wn, lane);
    }
    mfma_step<DT>(acc, f1);
  }
  // the reload that stood in for a missing slab may still be on its way into LDS: it is long
  // done by now, the wait only makes that explicit for whoever touches the buffers next
  if (!A_REG) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
__device__ __forceinline__ int64_t xcd_contiguous(int64_t wg, int64_t n) {
  const int64_t per = (n + 7) / 8;
  const int64_t t = (wg & 7) * per + (wg >> 3);
  return t;  // may be >= n for the last XCD's slack: callers skip those
}

// Work item t of a tiles_m x tiles_n grid -> (tm, tn) such that 32 consecutive items (what one
// XCD runs at a time) form an 8 x 4 block: 12 distinct operand row-blocks for 32 tiles, so most
// slab loads hit that XCD's L2.
__device__ __forceinline__ void grouped_tile(int64_t t, int64_t tiles_m, int64_t tiles_n, int64_t& tm, int64_t& tn) {
  const int64_t per_group = 8 * tiles_n;
  const int64_t group = t / per_group, in_group = t - group * per_group;
  const int64_t first = group * 8;
  const int64_t height = tiles_m - first < 8 ? tiles_m - first : 8;
  tn = in_group / height;
  tm = first + (in_group - tn * height);
}

}  // namespace mm
}  // namespace orlhf
