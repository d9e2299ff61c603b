// Decode GEMV for one to four token rows on gfx950 with every request of a wave in flight before anything is consumed.
//
// Same arithmetic and the same canonical buffers as the wave-dot GEMV (gemv.hip): a wave owns row blocks of two
// consecutive output rows and their whole K extent, lane l handles the 16-byte units l, l+64, ... of each row, codes
// are used in place as fp16 subnormals with v_dot2_f32_f16, the zero-point is folded through per-unit activation sums,
// and the correction rides along as a K-extension  y = [deq(W) | L] . [x ; alpha r].
//
// What differs is the memory schedule.  A wave handles one row block and issues ALL its loads (weights, scales,
// zero-point words, L rows) at its head, right behind the loads of the activations; it then stages the activations,
// meets the other waves at the one barrier, and consumes the row block in the order the data returns.  The memory
// pipe has the wave's whole work from the first microsecond on, instead of one step at a time behind a round trip
// each.  The loads are written as inline assembly so that the waits can be exact: the compiler's own wait insertion
// cannot see across the staging and falls back to waiting for everything (measured: a ring of prefetch buffers in
// plain C++ got slower with every added buffer for that reason).  Vector memory loads return in order, so
// "vmcnt(n)" with n = the number of loads issued behind the wanted one is exact; stores only make it conservative.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "side_stream.hpp"

namespace glowq {

// gemv.hip: LDS layout of the staged activations, shared by both single-row kernels
size_t wave_dot_lds_bytes(int M, int K, int rank, bool has_r);

namespace {

constexpr int kSRows = 2;  // rows per row block

// f(integral_constant<int, 0>) ... f(integral_constant<int, kN - 1>): loop indices usable as template arguments
template <int... kI, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, kI...>, F&& f) {
  (f(std::integral_constant<int, kI>{}), ...);
}
template <int kN, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, kN>{}, f);
}

__device__ __forceinline__ u32x4 ld_b128_nt(const void* sbase, uint32_t voff) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ u32x4 ld_b128(const void* sbase, uint32_t voff) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t ld_b32(const void* sbase, uint32_t voff) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t ld_b32_nt(const void* sbase, uint32_t voff) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
__device__ __forceinline__ u32x2 ld_b64_nt(const void* sbase, uint32_t voff) {
  u32x2 v;
  asm volatile("global_load_dwordx2 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ u32x3 ld_b96_nt(const void* sbase, uint32_t voff) {
  u32x3 v;
  asm volatile("global_load_dwordx3 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t ld_u16_nt(const void* sbase, uint32_t voff) {
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
// Waits until at most kN vector memory operations are outstanding; the registers named are the ones whose loads this
// wait is for (tying them to the statement keeps their first use behind it).
template <int kN>
__device__ __forceinline__ void wait_vm(u32x4& a, u32x4& b) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(kN) : "memory");
}
// The same with the index the step's LDS reads are addressed with: the reads of all steps would otherwise be hoisted
// to the top of the row block and held in registers (20 VGPRs per step).
template <int kN>
__device__ __forceinline__ void wait_vm(u32x4& a, u32x4& b, int& idx) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%3)" : "+v"(a), "+v"(b), "+v"(idx) : "n"(kN) : "memory");
}
template <int kN>
__device__ __forceinline__ void wait_vm(uint32_t& a) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(kN) : "memory");
}
template <int kN>
__device__ __forceinline__ void wait_vm(u32x2& a) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(kN) : "memory");
}
template <int kN>
__device__ __forceinline__ void wait_vm(u32x3& a) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(kN) : "memory");
}
template <int kN>
__device__ __forceinline__ void wait_vm(u32x4& a) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(kN) : "memory");
}

__device__ __forceinline__ void dot_word2(uint32_t w, const h8& xq, float& accA, float& accB) {
  // nibbles (0,4) and (2,6) land in mantissa bits 0-3, nibbles (1,5) and (3,7) in bits 4-7
  const uint32_t hi = w >> 8;
  accA = __builtin_amdgcn_fdot2(bitcast_u32<h2>(w & 0x000F000Fu), h2{xq[0], xq[1]}, accA, false);
  accB = __builtin_amdgcn_fdot2(bitcast_u32<h2>(w & 0x00F000F0u), h2{xq[2], xq[3]}, accB, false);
  accA = __builtin_amdgcn_fdot2(bitcast_u32<h2>(hi & 0x000F000Fu), h2{xq[4], xq[5]}, accA, false);
  accB = __builtin_amdgcn_fdot2(bitcast_u32<h2>(hi & 0x00F000F0u), h2{xq[6], xq[7]}, accB, false);
}

// What a wave holds of one row block: kKit steps of two 16-byte units (32 codes of each row), and the side data.
// From the canonical buffers: the scale and the zero-point word of one (row, group) per lane and pair of steps -- lane
// 32 r + i has group gbase(p) + i of row r for pair p -- and kLW dwords of each row of L.  From a side stream
// (side_stream.hpp) the same in kDwords = kNP + 2 kLW dwords per lane, fetched as chunks of up to four.
template <int kSize>
struct SideChunk;
template <>
struct SideChunk<1> { uint32_t v; __device__ __forceinline__ uint32_t get(int) const { return v; } };
template <>
struct SideChunk<2> { u32x2 v; __device__ __forceinline__ uint32_t get(int i) const { return v[i]; } };
template <>
struct SideChunk<3> { u32x3 v; __device__ __forceinline__ uint32_t get(int i) const { return v[i]; } };
template <>
struct SideChunk<4> { u32x4 v; __device__ __forceinline__ uint32_t get(int i) const { return v[i]; } };

template <int kKit, int kLW, bool kPacked>
struct SlotCounts {
  static constexpr int kNP = (kKit + 1) / 2;
  static constexpr int kDwords = kNP + kSRows * kLW;
  static constexpr int kFull = kDwords / 4, kTail = kDwords % 4;
  static constexpr int kSide = kPacked ? kFull + (kTail ? 1 : 0) : 2 * kNP + kSRows * kLW;  // loads ahead of the weights
  static constexpr int kLoads = kSide + kSRows * kKit;                                     // loads per row block
};
template <int kKit, int kLW, bool kPacked>
struct Slot {
  using C = SlotCounts<kKit, kLW, kPacked>;
  u32x4 w[kKit][kSRows];
  // canonical buffers
  uint32_t sc[kPacked ? 1 : C::kNP], zw[kPacked ? 1 : C::kNP];
  uint32_t l[kSRows][(!kPacked && kLW > 0) ? kLW : 1];
  // side stream
  SideChunk<4> q[(kPacked && C::kFull > 0) ? C::kFull : 1];
  SideChunk<(C::kTail ? C::kTail : 1)> tail;
  __device__ __forceinline__ uint32_t side(int d) const { return d < 4 * C::kFull ? q[d >> 2].get(d & 3) : tail.get(d & 3); }
};

// Heavy instantiations (more than four steps in flight per wave) run with at most 8 waves per workgroup, which leaves
// them 256 VGPRs, and fetch up to eight 16-byte words of each token row of x per thread; the others up to four.
__host__ __device__ constexpr bool stream_heavy(int kit) { return kit > 4; }
__host__ __device__ constexpr int stream_xw(int kit) { return stream_heavy(kit) ? 8 : 4; }

// kKit: steps (2048 columns) per row block; kLW: dwords of a row of L per lane (rank <= 128 kLW); kM: token rows (1..4),
// all served by the one pass over the weights: the masked code words are shared, only the dot products repeat per row.
// A wave handles ONE row block: the dispatcher hands out workgroups as others finish, which levels the end of the
// launch, and short waves leave more of them resident (two and four row blocks per wave measured 1.3 and 5 us slower
// on 28672 rows).
// Registers: a row block in flight is 8 kKit + 2 kNP + 2 kLW VGPRs that must never be spilled (a spill would store them
// before their loads have returned); the build checks that no instantiation uses scratch.  Light instantiations are
// held to 128 VGPRs (4 waves per SIMD), heavy ones get 256.
template <int kKit, int kLW, int kM, bool kPacked>
__global__ __launch_bounds__(stream_heavy(kKit) ? 512 : 1024)
__attribute__((amdgpu_waves_per_eu((stream_heavy(kKit) ? 1 : 2), (stream_heavy(kKit) ? 2 : 4))))
void gemv_stream_kernel(const half_t* __restrict__ x, const half_t* __restrict__ r, const int K, const int rank,
                        const int group_size, const float alpha, const GroupDev g) {
  using C = SlotCounts<kKit, kLW, kPacked>;
  constexpr int kNP = C::kNP;
  constexpr int kXW = stream_xw(kKit);
  static_assert(C::kLoads <= 63, "the wait for the activations counts every load behind them");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int U = K >> 5;
  const int upg_shift = __builtin_ctz(group_size >> 5);
  const int G = (U + (1 << upg_shift) - 1) >> upg_shift;
  // LDS: xs [kM][4][U] units of 8 halves in nibble order, sig [kM][U] = 2^-24 * sum of the unit, rs [kM][rank]
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + (size_t)kM * K * sizeof(half_t));
  half_t* rs = reinterpret_cast<half_t*>(smem + (((size_t)kM * K * sizeof(half_t) + (size_t)kM * U * sizeof(float) + 15) & ~(size_t)15));
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int threads = blockDim.x, waves = threads >> 6;
  const int ldw_half = rank >> 1;  // dwords per row of L

  // ---- activations first: their wait then does not cover the weight requests issued behind them
  const int words = K >> 3;
  u32x4 xw[kM][kXW];
  uint32_t rw[kM];
#pragma unroll
  for (int m = 0; m < kM; ++m) {
#pragma unroll
    for (int i = 0; i < kXW; ++i)
      xw[m][i] = ld_b128(x + (size_t)m * K, (uint32_t)min((int)threadIdx.x + i * threads, words - 1) * 16u);
    rw[m] = 0;
    if (kLW > 0) rw[m] = ld_b32(r + (size_t)m * rank, (uint32_t)min((int)threadIdx.x, ldw_half - 1) * 4u);
  }

  // ---- member of this workgroup (one round trip to the argument buffer, overlapped with the loads above)
  MemberDev mem = g.mem[0];
  int wg_begin = 0, total_blocks = g.task_end[0];
#define GLOWQ_PICK(i)                                            \
  if (g.n_members > i && (int)blockIdx.x >= g.wg_end[i - 1]) {  \
    mem = g.mem[i];                                              \
    wg_begin = g.wg_end[i - 1];                                  \
    total_blocks = g.task_end[i] - g.task_end[i - 1];            \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int want = ((int)blockIdx.x - wg_begin) * waves + wave;
  const bool valid = want < total_blocks;
  const int blk = valid ? want : total_blocks - 1;
  const float alpha_scaled = (mem.L != nullptr ? alpha : 0.f) * 0x1p-24f;  // accumulators carry 2^-24

  // ---- per-lane byte offsets
  // a wave past the member's last row block still issues its loads (the wait counts stay what they are), all lanes on
  // one address
  const uint32_t live = valid ? 0xFFFFFFFFu : 0u;
  const uint32_t voff = ((uint32_t)lane * 16u) & live;
  const int last_units = U - (kKit - 1) * kWave;                    // units of the last step (1..64)
  const uint32_t voff_last = ((uint32_t)min(lane, last_units - 1) * 16u) & live;
  const uint32_t rsel = (uint32_t)lane >> 5, gsel = (uint32_t)lane & 31u;
  // lane 32 r + i holds the scale and zero-point of group gbase(p) + i of row r for the pair of steps p, gbase(p) being
  // the first group of step 2 p (a pair of steps spans 128 units = 32 groups of 128 columns, fewer of larger groups)
  uint32_t sgrp[kNP];
#pragma unroll
  for (int p = 0; p < kNP; ++p) sgrp[p] = (uint32_t)min((int)(((128 * p) >> upg_shift) + gsel), G - 1);

  // ---- every load of the row block
  Slot<kKit, kLW, kPacked> b;
  {
    const int n0 = blk * kSRows;
    const bool two = n0 + 1 < mem.N;  // the second row exists
    const char* w0 = reinterpret_cast<const char*>(mem.qweight + (size_t)n0 * mem.ldw);
    const char* w1 = two ? w0 + (size_t)mem.ldw * 4 : w0;
    if constexpr (kPacked) {
      const char* sb = reinterpret_cast<const char*>(mem.side) + (size_t)blk * (256 * C::kDwords);
#pragma unroll
      for (int c = 0; c < C::kFull; ++c) b.q[c].v = ld_b128_nt(sb + 1024 * c, voff);
      if constexpr (C::kTail == 1) b.tail.v = ld_b32_nt(sb + 1024 * C::kFull, ((uint32_t)lane * 4u) & live);
      if constexpr (C::kTail == 2) b.tail.v = ld_b64_nt(sb + 1024 * C::kFull, ((uint32_t)lane * 8u) & live);
      if constexpr (C::kTail == 3) b.tail.v = ld_b96_nt(sb + 1024 * C::kFull, ((uint32_t)lane * 12u) & live);
    } else {
      const char* sc0 = reinterpret_cast<const char*>(mem.scales + (size_t)n0 * mem.lds);
      const char* zw0 = reinterpret_cast<const char*>(mem.qzeros + (size_t)n0 * mem.ldz);
      const uint32_t sc_row = two ? (uint32_t)mem.lds * 2u : 0u, zw_row = two ? (uint32_t)mem.ldz * 4u : 0u;
#pragma unroll
      for (int p = 0; p < kNP; ++p) {
        b.sc[p] = ld_u16_nt(sc0, (rsel * sc_row + sgrp[p] * 2u) & live);
        b.zw[p] = ld_b32_nt(zw0, (rsel * zw_row + (sgrp[p] >> 3) * 4u) & live);
      }
      if constexpr (kLW > 0) {
        // a member without L reads r itself (valid memory) and is weighted by zero
        const char* l0 = mem.L ? reinterpret_cast<const char*>(mem.L + (size_t)n0 * rank) : reinterpret_cast<const char*>(r);
        const char* l1 = (mem.L && two) ? l0 + (size_t)rank * 2 : l0;
#pragma unroll
        for (int j = 0; j < kLW; ++j) {
          const uint32_t lo = ((uint32_t)min(lane + kWave * j, ldw_half - 1) * 4u) & live;
          b.l[0][j] = ld_b32_nt(l0, lo);
          b.l[1][j] = ld_b32_nt(l1, lo);
        }
      }
    }
#pragma unroll
    for (int it = 0; it < kKit; ++it) {
      const uint32_t vo = it == kKit - 1 ? voff_last : voff;
      b.w[it][0] = ld_b128_nt(w0 + it * 1024, vo);
      b.w[it][1] = ld_b128_nt(w1 + it * 1024, vo);
    }
  }

  // ---- stage the activations (every load of x and r lies ahead of the row block's: one count covers them all)
#pragma unroll
  for (int m = 0; m < kM; ++m) {
#pragma unroll
    for (int i = 0; i < kXW; i += 2) wait_vm<C::kLoads>(xw[m][i], xw[m][i + 1]);
#pragma unroll
    for (int i = 0; i < kXW; ++i) {
      if (i * threads >= words) break;  // uniform: the words of this round lie past the row for every thread
      const int w = (int)threadIdx.x + i * threads;
      const h8 v = __builtin_bit_cast(h8, xw[m][i]);
      // sum of the eight halves: four dot products with (1, 1), fp32 accumulate
      const h2 ones = {(half_t)1.f, (half_t)1.f};
      float s = __builtin_amdgcn_fdot2(h2{v[0], v[1]}, ones, 0.f, false);
      s = __builtin_amdgcn_fdot2(h2{v[2], v[3]}, ones, s, false);
      s = __builtin_amdgcn_fdot2(h2{v[4], v[5]}, ones, s, false);
      s = __builtin_amdgcn_fdot2(h2{v[6], v[7]}, ones, s, false);
      s = quad_sum(s);  // threads and words are multiples of 4: a quad lies inside the row or outside as a whole
      if (w < words) {
        h8 p;
        p[0] = v[0]; p[1] = v[4]; p[2] = v[1]; p[3] = v[5];
        p[4] = v[2]; p[5] = v[6]; p[6] = v[3]; p[7] = v[7];
        const int u = w >> 2, j = w & 3;
        xs[((size_t)m * 4 + j) * U + u] = p;
        if (j == 0) sig[m * U + u] = s * 0x1p-24f;
      }
    }
    if constexpr (kLW > 0) {
      wait_vm<C::kLoads>(rw[m]);
      if ((int)threadIdx.x < ldw_half) reinterpret_cast<uint32_t*>(rs + (size_t)m * rank)[threadIdx.x] = rw[m];
    }
  }
  __syncthreads();
  if (!valid) return;  // (after the barrier; the loads still in flight land in registers nobody reads)

  // ---- consume the row block in the order it was requested
  float tot[kSRows][kM];
#pragma unroll
  for (int rr = 0; rr < kSRows; ++rr)
#pragma unroll
    for (int m = 0; m < kM; ++m) tot[rr][m] = 0.f;
  uint32_t rec = 0;
  static_for<kKit>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    constexpr int p = it >> 1;
    constexpr int kBehind = kSRows * (kKit - 1 - it);  // loads issued behind the weights of this step
    const int uraw = lane + it * kWave;
    const bool active = uraw < U;
    int u = active ? uraw : U - 1;
    if constexpr (it == 0) {
      // the side loads of a row block sit ahead of its weights: the same count covers them
      if constexpr (kPacked) {
#pragma unroll
        for (int c = 0; c < C::kFull; ++c) wait_vm<kBehind>(b.q[c].v);
        if constexpr (C::kTail > 0) wait_vm<kBehind>(b.tail.v);
      } else {
#pragma unroll
        for (int q = 0; q < kNP; ++q) {
          wait_vm<kBehind>(b.sc[q]);
          wait_vm<kBehind>(b.zw[q]);
        }
#pragma unroll
        for (int j = 0; j < kLW; ++j) {
          wait_vm<kBehind>(b.l[0][j]);
          wait_vm<kBehind>(b.l[1][j]);
        }
      }
    }
    wait_vm<kBehind>(b.w[it][0], b.w[it][1], u);
    const int grp = u >> upg_shift;
    if constexpr ((it & 1) == 0) {
      if constexpr (kPacked) rec = b.side(p);
      else rec = (b.sc[p] & 0xFFFFu) | (nibble(b.zw[p], (int)(sgrp[p] & 7u)) << 16);
    }
    float sc[kSRows], zp[kSRows];
    const int grel = grp - ((128 * p) >> upg_shift);
#pragma unroll
    for (int rr = 0; rr < kSRows; ++rr) {
      const uint32_t sv = (uint32_t)__builtin_amdgcn_ds_bpermute((32 * rr + grel) << 2, (int)rec);
      sc[rr] = active ? (float)__builtin_bit_cast(half_t, (uint16_t)(sv & 0xFFFFu)) : 0.f;
      zp[rr] = (float)(sv >> 16);
    }
    // the masked code words of the step, shared by every token row
    uint32_t cw[kSRows][4][4];
#pragma unroll
    for (int rr = 0; rr < kSRows; ++rr)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w = b.w[it][rr][q], hi = w >> 8;
        cw[rr][q][0] = w & 0x000F000Fu;   // nibbles (0,4): mantissa bits 0-3
        cw[rr][q][1] = w & 0x00F000F0u;   // nibbles (1,5): bits 4-7
        cw[rr][q][2] = hi & 0x000F000Fu;  // nibbles (2,6)
        cw[rr][q][3] = hi & 0x00F000F0u;  // nibbles (3,7)
      }
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      h8 xq[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) xq[j] = xs[((size_t)m * 4 + j) * U + u];
      const float sg = sig[m * U + u];
#pragma unroll
      for (int rr = 0; rr < kSRows; ++rr) {
        float accA = 0.f, accB = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          accA = __builtin_amdgcn_fdot2(bitcast_u32<h2>(cw[rr][q][0]), h2{xq[q][0], xq[q][1]}, accA, false);
          accB = __builtin_amdgcn_fdot2(bitcast_u32<h2>(cw[rr][q][1]), h2{xq[q][2], xq[q][3]}, accB, false);
          accA = __builtin_amdgcn_fdot2(bitcast_u32<h2>(cw[rr][q][2]), h2{xq[q][4], xq[q][5]}, accA, false);
          accB = __builtin_amdgcn_fdot2(bitcast_u32<h2>(cw[rr][q][3]), h2{xq[q][6], xq[q][7]}, accB, false);
        }
        float v = __builtin_fmaf(accB, 0.0625f, accA);
        v = __builtin_fmaf(-zp[rr], sg, v);
        tot[rr][m] = __builtin_fmaf(sc[rr], v, tot[rr][m]);
      }
    }
    if constexpr (it == 0 && kLW > 0) {
#pragma unroll
      for (int j = 0; j < kLW; ++j) {
        const int idx = lane + kWave * j;
        const float a = idx < ldw_half ? alpha_scaled : 0.f;
#pragma unroll
        for (int m = 0; m < kM; ++m) {
          const h2 rv = reinterpret_cast<const h2*>(rs + (size_t)m * rank)[min(idx, ldw_half - 1)];
#pragma unroll
          for (int rr = 0; rr < kSRows; ++rr)
            tot[rr][m] = __builtin_fmaf(a, __builtin_amdgcn_fdot2(bitcast_u32<h2>(kPacked ? b.side(kNP + kSRows * j + rr) : b.l[rr][j]),
                                                               rv, 0.f, false), tot[rr][m]);
        }
      }
    }
    // The step's sums are pinned here (an empty statement that "rewrites" them): left alone, the compiler sinks the whole
    // arithmetic of every step to the point of the reduction below, behind all the waits, and keeps every loaded word
    // and activation fragment of every step live until then (30 VGPRs per step and token row).
#pragma unroll
    for (int rr = 0; rr < kSRows; ++rr)
#pragma unroll
      for (int m = 0; m < kM; ++m) asm volatile("" : "+v"(tot[rr][m]));
  });
  // lane rr keeps the total of row rr: one store (and one bias load) per token row
  const int n = blk * kSRows + lane;
  const bool writer = lane < kSRows && n < mem.N;
  const float bias = (writer && mem.bias) ? (float)mem.bias[n] : 0.f;
#pragma unroll
  for (int m = 0; m < kM; ++m) {
    // both rows at once: a swap of the upper half of row 0's register with the lower half of row 1's leaves lanes
    // 0..31 with row 0 (lane l and lane l + 32 added) and lanes 32..63 with row 1; four DPP steps then sum every row of
    // 16 lanes, and the two 16-lane totals of each half meet through scalar lane reads
    // (inline assembly: this compiler's builtin for the swap loses its second result -- it added the first to itself;
    // the no-ops are the wait states a VALU result needs before the swap and the swap's results before DPP use)
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(tot[0][m]), "+v"(tot[1][m]));
    float v = tot[0][m] + tot[1][m];
    int t;
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true);  // row_half_mirror
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true);  // row_mirror
    v += __builtin_bit_cast(float, t);
    const int iv = __builtin_bit_cast(int, v);
    const float row0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    const float row1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    const float mine = lane == 0 ? row0 : row1;
    if (writer) mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(mine, 0x1p24f, bias));
  }
}

}  // namespace

// ---- host side ---------------------------------------------------------------------------------------------
// The stream GEMV takes up to four token rows on the fast layout with quantisation groups of 128 columns and more (a
// pair of steps then holds at most 32 groups of a row: one per lane of a half wave), K up to 9 steps of 2048 columns,
// ranks up to 256, and activations that the workgroup can fetch in four (eight) requests per thread and token row.
bool stream_supported(const GroupDev& g) {
  if (g.M < 1 || g.M > 4 || (g.K & 31) != 0 || g.K > 9 * 2048) return false;
  if (g.group_size < 128 || (g.group_size & (g.group_size - 1)) != 0) return false;
  const bool has_r = g.r != nullptr;
  if (has_r && ((g.rank & 1) != 0 || g.rank > 256 || g.rank < 2 || (reinterpret_cast<uintptr_t>(g.r) & 3u) != 0)) return false;
  if ((reinterpret_cast<uintptr_t>(g.x) & 15u) != 0) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if ((reinterpret_cast<uintptr_t>(m.qweight) & 15u) != 0 || (m.ldw & 3) != 0) return false;
    if (m.L && (reinterpret_cast<uintptr_t>(m.L) & 3u) != 0) return false;
    // 32-bit byte offsets inside every buffer of a member
    if ((long)m.N * m.ldw * 4 >= (1L << 31)) return false;
  }
  return wave_dot_lds_bytes(g.M, g.K, g.rank, has_r) <= 160 * 1024;
}

namespace {

template <int kKit, int kLW, int kM, bool kPacked>
hipError_t launch_stream_p(GroupDev& g, int waves, hipStream_t stream) {
  {
    auto kern = gemv_stream_kernel<kKit, kLW, kM, kPacked>;
    const size_t lds = wave_dot_lds_bytes(kM, g.K, g.rank, g.r != nullptr);
    static LdsLimit lds_limit;
    if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
    int total = 0, grid = 0;
    for (int i = 0; i < g.n_members; ++i) {
      const int blocks = (g.mem[i].N + kSRows - 1) / kSRows;
      total += blocks;
      g.task_end[i] = total;
      grid += (blocks + waves - 1) / waves;
      g.wg_end[i] = grid;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * kWave), lds, stream, g.x, g.r, g.K, g.r ? g.rank : 0, g.group_size,
                       g.alpha, g);
    return hipGetLastError();
  }
}

template <int kKit, int kLW>
hipError_t launch_stream_m(GroupDev& g, int waves, hipStream_t stream) {
  bool packed = true;
  for (int i = 0; i < g.n_members; ++i) packed = packed && g.mem[i].side != nullptr;
  switch (g.M) {
    case 1: return packed ? launch_stream_p<kKit, kLW, 1, true>(g, waves, stream) : launch_stream_p<kKit, kLW, 1, false>(g, waves, stream);
    case 2: return launch_stream_p<kKit, kLW, 2, false>(g, waves, stream);  // side streams serve single rows only
    case 3: return launch_stream_p<kKit, kLW, 3, false>(g, waves, stream);
    case 4: return launch_stream_p<kKit, kLW, 4, false>(g, waves, stream);
    default: return hipErrorInvalidValue;
  }
}

template <int kKit>
hipError_t launch_stream_lw(GroupDev& g, int waves, hipStream_t stream) {
  const int lw = g.r ? (g.rank + 127) / 128 : 0;
  if (lw == 0) return launch_stream_m<kKit, 0>(g, waves, stream);
  if (lw == 1) return launch_stream_m<kKit, 1>(g, waves, stream);
  return launch_stream_m<kKit, 2>(g, waves, stream);
}

int env_int_s(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

}  // namespace

hipError_t launch_stream(GroupDev& g, int num_cus, hipStream_t stream) {
  (void)num_cus;
  const int U = g.K >> 5;
  const int kit = (U + kWave - 1) / kWave;
  long blocks = 0;
  for (int i = 0; i < g.n_members; ++i) blocks += (g.mem[i].N + kSRows - 1) / kSRows;
  // 4 waves per workgroup, 8 for the long groups (measured: q|k|v 5.1 us at 4 against 5.6 at 8, down_proj 8.7 against 9.5,
  // gate|up 13.5 against 13.3)
  static const int env_waves = env_int_s("GLOWQ_STREAM_WAVES", 0);
  // (with more than one token row the long-K instantiations want 8 as well: down_proj at three rows 13.4 us against 18.2)
  int waves = env_waves > 0 ? env_waves : ((blocks >= 8192 || (g.M > 1 && stream_heavy(kit))) ? 8 : 4);
  const int max_waves = stream_heavy(kit) ? 8 : 16;
  if (waves > max_waves) waves = max_waves;
  while ((g.K >> 3) > stream_xw(kit) * waves * kWave && waves < max_waves) ++waves;
  if ((g.K >> 3) > stream_xw(kit) * waves * kWave) return hipErrorInvalidValue;
  switch (kit) {
    case 1: return launch_stream_lw<1>(g, waves, stream);
    case 2: return launch_stream_lw<2>(g, waves, stream);
    case 3: return launch_stream_lw<3>(g, waves, stream);
    case 4: return launch_stream_lw<4>(g, waves, stream);
    case 5: return launch_stream_lw<5>(g, waves, stream);
    case 6: return launch_stream_lw<6>(g, waves, stream);
    case 7: return launch_stream_lw<7>(g, waves, stream);
    case 8: return launch_stream_lw<8>(g, waves, stream);
    case 9: return launch_stream_lw<9>(g, waves, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace glowq
