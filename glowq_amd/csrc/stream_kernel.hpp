// The stream GEMV kernel (gfx950): one to four token rows, every request of a wave in flight before anything is
// consumed.  Included by gemv_stream.hip (the plain group launch) and gemv_chain.hip (the single-token forms that take
// over the work between two linears of a decoder layer).
//
// Same arithmetic and the same canonical buffers as the wave-dot GEMV (gemv.hip): a wave owns a row block of two output
// rows and their whole K extent, lane l handles the 16-byte units l, l+64, ... of each row, codes are used in place as
// fp16 subnormals with v_dot2_f32_f16, the zero-point is folded through per-unit activation sums, and the correction
// rides along as a K-extension  y = [deq(W) | L] . [x ; alpha r].
//
// What differs is the memory schedule.  A wave handles one row block and issues ALL its loads (weights, scales,
// zero-point words, L rows) at its head, right behind the loads of the activations; it then stages the activations,
// meets the other waves at the one barrier, and consumes the row block in the order the data returns.  The memory
// pipe has the wave's whole work from the first microsecond on, instead of one step at a time behind a round trip
// each.  The loads are written as inline assembly so that the waits can be exact: the compiler's own wait insertion
// cannot see across the staging and falls back to waiting for everything (measured: a ring of prefetch buffers in
// plain C++ got slower with every added buffer for that reason).  Vector memory loads return in order, so
// "vmcnt(n)" with n = the number of loads issued behind the wanted one is exact; memory operations the compiler adds
// on its own only make it conservative.
#pragma once

#include <type_traits>
#include <utility>

#include "common.hpp"
#include "handover.hpp"
#include "side_stream.hpp"

namespace glowq {
namespace streamk {

constexpr int kSRows = 2;  // rows per row block

// ---- chained forms (single token) ---------------------------------------------------------------------------------
// Between two linears of a decoder layer sit a residual add, an RMSNorm or a SwiGLU gate, and the projection of the
// result on the next group's right factor.  The chained forms move that work into the two launches on either side:
//
//   epilogue of the producer   kEpiResidual: x_res[n] = fp16(x_res[n] + y[n]) for the wave's own rows, and their share
//                                of  P = R_next (w_next (.) x_res)  (w_next: weight of the norm that follows);
//                              kEpiSwiglu: the wave's two rows are row n of gate and row n of up, act[n] =
//                                fp16(fp16(silu(gate)) * up), and its share of  P = R_next act.
//   prologue of the consumer   kProAcc: r = fp16(P);  kProNormAcc: the workgroup computes the norm factor
//                                f = rsqrt(mean(x_res^2) + eps) itself, stages h = fp16(fp16(x_res f) w) and takes
//                                r = fp16(f P)  (the norm is linear in x_res up to that one scalar).
//
// P travels through an accumulator in device memory: kAccCopies x kAccStride 64-bit integers, fixed point with 32
// fractional bits.  A workgroup sums the shares of its waves in LDS in wave order and adds the total, rounded to fixed
// point, to copy (workgroup index mod kAccCopies) with one integer atomic per entry; the consumer adds up the copies.
// Integer addition is associative, so the result does not depend on the order in which workgroups arrive: the chain is
// as reproducible as the separate kernels it replaces.  The word behind the copies is an overflow flag: a workgroup
// whose partial sum is not below the limit it was given (2^31 / number of workgroups; any NaN) sets it, and the consumer
// then takes r = NaN instead of a wrapped sum.  The accumulator must be zero (flag included) when the producer starts.
// (ChainDev and the constants: common.hpp)

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
__device__ __forceinline__ u32x2 ld_b64(const void* sbase, uint32_t voff) {
  u32x2 v;
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ u32x2 ld_b64_nt(const void* sbase, uint32_t voff) {
  u32x2 v;
  asm volatile("global_load_dwordx2 %0, %1, %2 nt" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
// (a relaxed atomic load of agent scope: past the caches that are private to a part of the chip)
__device__ __forceinline__ u32x2 ld_b64_agent(const void* sbase, uint32_t voff) {
  u32x2 v;
  asm volatile("global_load_dwordx2 %0, %1, %2 sc1" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
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
// The same with a full address per lane (the two rows of a gate/up pair lie in different buffers).
__device__ __forceinline__ uint32_t ld_u16_nt_at(const void* vaddr) {
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, off nt" : "=v"(v) : "v"(vaddr) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t ld_b32_nt_at(const void* vaddr) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off nt" : "=v"(v) : "v"(vaddr) : "memory");
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
__device__ __forceinline__ void wait_vm(u32x4& a, int& idx) {
  static_assert(kN >= 0 && kN <= 63, "vmcnt is a 6-bit field");
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(idx) : "n"(kN) : "memory");
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

// The same for an array of 1, 2, 4 or 8 words.
template <int kN, int kCount>
__device__ __forceinline__ void wait_words(u32x4 (&a)[kCount]) {
  static_assert(kCount == 1 || (kCount & 1) == 0, "one word or pairs of words");
  if constexpr (kCount == 1) {
    wait_vm<kN>(a[0]);
  } else {
#pragma unroll
    for (int i = 0; i < kCount; i += 2) wait_vm<kN>(a[i], a[i + 1]);
  }
}

// ---- the projection inside the launch (kProProj, single token) -----------------------------------------------------
// r = R x is needed by every wave, but only for the last of its dot products.  Instead of a launch of its own in front
// (2.4 to 3.4 us for 128 rows of R), the grid gets workgroups in front that have no row block: their waves compute the
// entries of r and hand them to everybody else through one 64-bit word per entry in device memory:
//     bits 48..63: the fp16 value,   bits 0..47: a tag that names this launch.
// Value and tag travel in the one word, written and read with relaxed atomics of agent scope (they pass the caches that
// are private to a part of the chip), so a reader that sees the tag has the value and no fence is needed.  The tag is
// built from the dispatch id of the launch -- the position of its packet in the hardware queue, which a replay of a
// captured graph renews like any other launch -- and from the address of that queue, with the top bit set so that
// zeroed memory never matches.  Words left by earlier launches therefore never pass for this launch's, and nothing has
// to be cleared between launches.  A reader looks at its word when the last of its weights are due; one that does not
// find the tag polls a bounded number of times and then computes its entry itself, so every wave ends whatever the
// order in which the workgroups were started.  Calls that share the words must not overlap.
// How the entries reach the block the readers look at depends on how many one workgroup produces.  With one wave per
// entry (up to 8192 columns) a workgroup's entries meet in LDS and one store writes them into the block, consecutive
// words.  With four waves per entry (longer rows: one or two entries per workgroup) a producer leaves its word in a
// staging area that only the collectors read: the waves of one more workgroup in front, which poll it in turn
// (bounded) until all entries of this launch are there; one of them then writes the block, 512 contiguous bytes per
// store instruction.  What matters is how often a line of the block is written while thousands of readers fetch it:
// every write sends the readers of all parts of the chip back to memory for the line.  128 producers writing eight
// bytes each straight into the block cost the launch 0.8 to 1.5 us; sixteen or eight bytes per workgroup (the long rows)
// were slower than the detour through the collectors (13.8 against 10.8 us); 32 bytes per workgroup are faster than
// the detour (q|k|v 6.75 against 7.05 us, o_proj 6.2 against 6.7), which costs a round trip of its own.
// What it buys is bounded by the hand-over itself: a row of R that no cache holds is there 2 to 2.5 us after the launch
// began, and each hop through memory adds half a microsecond or more, which together is about as long as the launch of
// a small group takes without it.  Per group launch of a 32-layer sequence, projection inside / projection launch in
// front / r given: q|k|v of an 8B layer 6.75 / 7.5 / 5.1 us, o_proj 6.3 / 6.7 / 4.3, down_proj 10.8 / 11.85 / 8.4; the
// whole layer 39.15 against 40.6.  (Tried on the way and slower: producers that also own a row block; a first look
// right behind the barrier, with or without a pause in front of it; 2 to 256 copies of the block for the readers to
// spread over; the lines of the block 4096 bytes apart.)
// The staging words lie 4096 bytes behind the block, not right behind it: next to each other, the collectors' polls and
// the readers' meet at the same place in memory (q|k|v of an 8B layer 7.45 us against 7.15).  (The lines of the block
// themselves 4096 bytes apart, to spread the readers: 7.35.)
constexpr int kProjStaging = 512;
__device__ __forceinline__ float dot8(const h8& a, const h8& c) {
  float d = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) d = __builtin_amdgcn_fdot2(h2{a[2 * i], a[2 * i + 1]}, h2{c[2 * i], c[2 * i + 1]}, d, false);
  return d;
}
// Entries of r in the summation order of the projection launch they stand in for (misc.hip), so that both ways give the
// same bits.  Up to 8192 columns one wave owns an entry: lane l adds the 16-byte pieces l, l + 64, ... in turn
// (shared_proj_wave_kernel).  Above, four waves share it like the four waves of the 256-thread kernel: wave q adds the
// pieces l + 64 q, l + 64 q + 256, ..., and the four wave totals meet as (p0 + p1) + (p2 + p3) (shared_proj_kernel<1>).
__host__ __device__ constexpr bool proj_split(int words) { return words > 1024; }
__host__ __device__ constexpr int proj_entries_per_wg(int words, int waves) { return proj_split(words) ? waves >> 2 : waves; }
// workgroups in front of the grid: those that produce r, and the collector's
__host__ __device__ constexpr int proj_front_wgs(int words, int waves, int rank) {
  return (rank + proj_entries_per_wg(words, waves) - 1) / proj_entries_per_wg(words, waves) + 1;
}

// What a wave holds of one row block: kKit steps of two 16-byte units (32 codes of each row), and the side data.
// From the canonical buffers: the scale and the zero-point word of one (row, group) per lane and pair of steps -- lane
// 32 r + i has group gbase(p) + i of row r for pair p -- and kLW dwords of each row of L.  From a side stream
// (side_stream.hpp) the same in kDwords = kNP + 2 kLW dwords per lane, fetched as chunks of up to four.  The chained
// epilogues add kLW dwords of each row of the next group's transposed right factor (one row for a gate/up pair).
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

__host__ __device__ constexpr int epi_rows(int epi) { return epi == kEpiResidual ? 2 : (epi == kEpiSwiglu ? 1 : 0); }

template <int kKit, int kLW, bool kPacked, int kEpi>
struct SlotCounts {
  static constexpr int kNP = (kKit + 1) / 2;
  static constexpr int kDwords = kNP + kSRows * kLW;
  static constexpr int kFull = kDwords / 4, kTail = kDwords % 4;
  static constexpr int kRt = epi_rows(kEpi) * kLW;  // loads of the next right factor
  static constexpr int kSide = (kPacked ? kFull + (kTail ? 1 : 0) : 2 * kNP + kSRows * kLW) + kRt;  // loads ahead of the weights
  static constexpr int kLoads = kSide + kSRows * kKit;                                            // loads per row block
};
template <int kKit, int kLW, bool kPacked, int kEpi>
struct Slot {
  using C = SlotCounts<kKit, kLW, kPacked, kEpi>;
  u32x4 w[kKit][kSRows];
  // canonical buffers
  uint32_t sc[kPacked ? 1 : C::kNP], zw[kPacked ? 1 : C::kNP];
  uint32_t l[kSRows][(!kPacked && kLW > 0) ? kLW : 1];
  // side stream
  SideChunk<4> q[(kPacked && C::kFull > 0) ? C::kFull : 1];
  SideChunk<(C::kTail ? C::kTail : 1)> tail;
  // next right factor
  uint32_t rt[kSRows][(kEpi != kEpiNone && kLW > 0) ? kLW : 1];
  __device__ __forceinline__ uint32_t side(int d) const { return d < 4 * C::kFull ? q[d >> 2].get(d & 3) : tail.get(d & 3); }
};

// Heavy instantiations (more than four steps in flight per wave) run with at most 8 waves per workgroup, which leaves
// them 256 VGPRs, and fetch up to eight 16-byte words of each token row of x per thread; the others up to four.
__host__ __device__ constexpr bool stream_heavy(int kit) { return kit > 4; }
__host__ __device__ constexpr int stream_xw(int kit) { return stream_heavy(kit) ? 8 : 4; }
// Waves per SIMD the register allocation aims at (the bounds of amdgpu_waves_per_eu).  The plain light forms end up at
// 64 VGPRs = 8 waves by themselves; the chained ones carry norm weights, accumulator words and the next right factor on
// top and have to be told (left at 4 waves the gate|up launch of an 8B layer took 23.7 us instead of 13): as many waves
// as compile without spilling -- the build refuses scratch in these kernels.  (The forms with the projection inside
// the launch come out one or two registers above 64 at up to two steps, and are held to 8 waves as well where they
// read side streams, to 7 from the canonical buffers.)
__host__ __device__ constexpr int stream_min_waves(int kit, int lw, int al, bool chained) {
  if (stream_heavy(kit)) return 1;
  if (!chained || kit > 2) return 2;
  return lw <= 1 ? (al <= 2 ? 8 : 7) : (al <= 2 ? 6 : 2);
}
__host__ __device__ constexpr bool stream_chained(int pro, int epi) { return pro == kProAcc || pro == kProNormAcc || epi != kEpiNone; }
__host__ __device__ constexpr int stream_max_waves(int kit, bool chained) { return stream_heavy(kit) ? 2 : (chained && kit <= 2 ? 8 : 4); }

// LDS of the plain forms: xs [kM][4][U] units of 8 halves in nibble order, sig [kM][U], rs [kM][rank] (gemv.hip); the
// chained forms add 16 floats for the norm's sum of squares, waves x 128 kLW 64-bit sums of the accumulator's copies
// and waves x rank floats for the shares of P.
__host__ __device__ constexpr size_t chain_extra_lds(int waves, int rank) {
  return 64 + (size_t)waves * 128 * ((rank + 127) / 128) * sizeof(long long) + (size_t)waves * rank * sizeof(float);
}
// Words of x per thread and loads of the accumulator per thread in the chained forms, by the least number of waves a
// workgroup is launched with (4 or 8): the fewer of both, the more waves a SIMD holds (registers, not LDS, bound it).
__host__ __device__ constexpr int chain_xw(int kit, bool w8) {
  const int need = (kit * 256 + (w8 ? 512 : 256) - 1) / (w8 ? 512 : 256);
  return need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
}
__host__ __device__ constexpr int chain_acc_loads(bool w8) { return w8 ? 2 : 4; }

// kKit: steps (2048 columns) per row block; kLW: dwords of a row of L per lane (rank <= 128 kLW); kM: token rows (1..4),
// all served by the one pass over the weights: the masked code words are shared, only the dot products repeat per row.
// kPro / kEpi: the chained forms (single token, canonical buffers).
// A wave handles ONE row block: the dispatcher hands out workgroups as others finish, which levels the end of the
// launch, and short waves leave more of them resident (two and four row blocks per wave measured 1.3 and 5 us slower
// on 28672 rows).
// Registers: a row block in flight is 8 kKit + 2 kNP + 2 kLW VGPRs that must never be spilled (a spill would store them
// before their loads have returned); the build checks that no instantiation uses scratch.  Light instantiations are
// held to 128 VGPRs (4 waves per SIMD), heavy ones get 256.
template <int kKit, int kLW, int kM, bool kPacked, int kPro, int kEpi, int kXW, int kAL>
__global__ __launch_bounds__(stream_heavy(kKit) ? 512 : 1024)
__attribute__((amdgpu_waves_per_eu(kPro == kProProj && kKit <= 2 ? (kPacked ? 8 : 7) : stream_min_waves(kKit, kLW, kAL, stream_chained(kPro, kEpi)),
                                   kPro == kProProj && kKit <= 2 ? 8 : stream_max_waves(kKit, stream_chained(kPro, kEpi)))))
void gemv_stream_kernel(const half_t* __restrict__ x, const half_t* __restrict__ r, const int K, const int rank,
                        const int group_size, const float alpha, const GroupDev g, const ChainDev ch) {
  using C = SlotCounts<kKit, kLW, kPacked, kEpi>;
  constexpr int kNP = C::kNP;
  constexpr bool kChained = stream_chained(kPro, kEpi);
  constexpr bool kAccPro = kPro == kProAcc || kPro == kProNormAcc;  // r comes out of an accumulator
  // kProProj: each thread's first look at its entry of r goes out ahead of the wait for the last step's weights
  constexpr int kLook = kPro == kProProj ? 1 : 0;
  static_assert(C::kLoads + kLook <= 63, "the waits count every load behind the one they are for");
  static_assert(!kChained || (kM == 1 && !kPacked), "the chained forms serve one token from the canonical buffers");
  static_assert(kPro == kProPlain || kLW > 0, "every other prologue is about r");
  static_assert(kPro != kProProj || (kM == 1 && kEpi == kEpiNone), "the projection inside the launch serves one token, plain epilogue");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int U = K >> 5;
  const int upg_shift = __builtin_ctz(group_size >> 5);
  const int G = (U + (1 << upg_shift) - 1) >> upg_shift;
  // LDS: xs [kM][4][U] units of 8 halves in nibble order, sig [kM][U] = 2^-24 * sum of the unit, rs [kM][rank]
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + (size_t)kM * K * sizeof(half_t));
  const size_t rs_off = ((size_t)kM * K * sizeof(half_t) + (size_t)kM * U * sizeof(float) + 15) & ~(size_t)15;
  half_t* rs = reinterpret_cast<half_t*>(smem + rs_off);
  // chained forms: red [16], accp [waves][128 kLW] 64-bit sums of the accumulator's copies, part [waves][rank]
  float* red = reinterpret_cast<float*>(smem + ((rs_off + (size_t)kM * rank * sizeof(half_t) + 15) & ~(size_t)15));
  long long* accp = reinterpret_cast<long long*>(red + 16);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int threads = blockDim.x, waves = threads >> 6;
  const int ldw_half = rank >> 1;  // dwords per row of L
  float* part = reinterpret_cast<float*>(accp + (kAccPro ? (size_t)waves * 128 * kLW : 0));

  const int words = K >> 3;
  // ---- kProProj: the workgroups in front of the grid have no row block (see above).  They are the first to be started
  // and nobody's weights wait behind their dot products.  Their waves produce one entry of r each and leave it in the
  // staging words; wave 0 of the last of them collects the staging words and publishes the block the readers look at.
  unsigned long long tag = 0;
  int wg = (int)blockIdx.x;
  if constexpr (kPro == kProProj) {
    tag = launch_tag();
    const int front = proj_front_wgs(words, waves, rank);
    unsigned long long* staging = ch.proj_pub + kProjStaging;
    // (roles in front go to the workgroup indices that start first: handover.hpp)
    const int role = front_role(wg, front);
    if (role >= front) return;
    if (role >= 0 && role < front - 1) {
      // the row of R first (up to eight pieces per lane in flight), then x into LDS in its natural order by the whole
      // workgroup while they travel
      const bool split = proj_split(words);
      const int epw = proj_entries_per_wg(words, waves);
      const int j = __builtin_amdgcn_readfirstlane(role * epw + (split ? wave >> 2 : wave));
      const int q = split ? wave & 3 : 0;
      const bool active = j < rank && (!split || wave < 4 * epw);
      const int stride = split ? 256 : kWave, first = lane + kWave * q;
      const int pieces = (words + stride - 1) / stride;  // of the lanes with the most
      // (a scalar base and 32-bit byte offsets: eight 64-bit addresses per lane would cost the kernel a wave per SIMD)
      const char* Rb = reinterpret_cast<const char*>(ch.proj_R + (size_t)(active ? j : 0) * K);
      auto piece = [&](int w) { return *reinterpret_cast<const h8*>(Rb + ((uint32_t)min(w, words - 1) << 4)); };
      h8* xn = reinterpret_cast<h8*>(smem);
      float* pp = reinterpret_cast<float*>(smem + (size_t)K * sizeof(half_t));  // (split form: K > 8192, room for 16 floats)
      // (one batch holds a whole share of the longest row the kernel takes: 9 pieces per lane where four waves share an
      // entry, which are the instantiations with registers to spare)
      constexpr int kBatch = stream_heavy(kKit) ? 9 : 8;
      h8 rv[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) rv[b] = piece(first + stride * b);
#pragma unroll 1
      for (int w = (int)threadIdx.x; w < words; w += threads) xn[w] = reinterpret_cast<const h8*>(x)[w];
      __syncthreads();
      float acc = 0.f;
      for (int b0 = 0; b0 < pieces; b0 += kBatch) {
        if (b0 > 0) {
#pragma unroll
          for (int b = 0; b < kBatch; ++b) rv[b] = piece(first + stride * (b0 + b));
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          const int w = first + stride * (b0 + b);
          const float d = dot8(rv[b], xn[min(w, words - 1)]);
          acc = w < words ? acc + d : acc;
        }
      }
      float total = wave_sum(acc);
      if (split) {
        if (lane == 0) pp[wave] = total;
        __syncthreads();
        total = (pp[wave & ~3] + pp[(wave & ~3) + 1]) + (pp[(wave & ~3) + 2] + pp[(wave & ~3) + 3]);
      }
      if (!split) {
        // one wave per entry: the workgroup's entries meet in LDS and go straight into the block the readers look at,
        // consecutive words in one store
        float* mine = reinterpret_cast<float*>(smem);  // (over the head of x, which every wave is done with behind the barrier)
        __syncthreads();
        if (lane == 0) mine[wave] = total;
        __syncthreads();
        if (wave == 0 && lane < epw && role * epw + lane < rank) {
          const half_t v = (half_t)mine[lane];
          ch.proj_r_out[role * epw + lane] = v;
          // (proj_mute: a test of the readers' own dot product -- the caller still gets r, the readers never do)
          if (!ch.proj_mute)
            __hip_atomic_store(ch.proj_pub + role * epw + lane, ((unsigned long long)__builtin_bit_cast(uint16_t, v) << 48) | tag,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
      }
      // four waves per entry: through the staging words and the collectors
      if (active && q == 0 && lane == 0) {
        const half_t v = (half_t)total;
        ch.proj_r_out[j] = v;
        if (!ch.proj_mute)
          __hip_atomic_store(staging + j, ((unsigned long long)__builtin_bit_cast(uint16_t, v) << 48) | tag, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      }
      return;
    }
    if (role == front - 1) {
      if (!proj_split(words)) return;  // (one wave per entry: the producers write the block themselves)
      // the collectors: the waves of this workgroup poll the staging words in turn, each a fraction of a round trip
      // behind the one before, so that the last entry is noticed soon after it lands.  The first wave to find all
      // entries of this launch claims the block through a flag in LDS and writes it -- once: a block written twice sends
      // the readers back to memory for it twice.  Lane l takes entries l, l + 64, ...: each store instruction below
      // writes 512 contiguous bytes, whole lines.
      int* claimed = reinterpret_cast<int*>(smem);
      if (threadIdx.x == 0) *claimed = 0;
      __syncthreads();
      for (int i = 0; i < wave; ++i) __builtin_amdgcn_s_sleep(6);
      unsigned long long w[4] = {0, 0, 0, 0};
      bool all = false;
      for (unsigned spins = 0; !all && spins <= ch.proj_spin; ++spins) {
        if (*reinterpret_cast<volatile int*>(claimed) != 0) return;
        bool mine = true;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (lane + kWave * q < rank) {
            w[q] = __hip_atomic_load(staging + lane + kWave * q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            mine = mine && (w[q] & kTagMask) == tag;
          }
        }
        all = __builtin_amdgcn_ballot_w64(!mine) == 0;
      }
      if (all) {
        int first = 0;
        if (lane == 0) first = atomicCAS(claimed, 0, 1) == 0;
        if (__builtin_amdgcn_readfirstlane(first)) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (lane + kWave * q < rank) __hip_atomic_store(ch.proj_pub + lane + kWave * q, w[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      return;  // (without all entries nothing is published: the readers run into their limit and compute r themselves)
    }
  }

  // ---- activations first: their wait then does not cover the weight requests issued behind them
  u32x4 xw[kM][kXW];
  u32x4 nw[kPro == kProNormAcc ? kXW : 1];
  uint32_t rw[kM];
  // accumulator: wave w takes copies w, w + waves, ...; lane l their entries 2 l, 2 l + 1 (+ 128 j)
  u32x4 av[kAccPro ? kAL : 1][kLW > 0 ? kLW : 1];
#pragma unroll
  for (int m = 0; m < kM; ++m) {
#pragma unroll
    for (int i = 0; i < kXW; ++i)
      xw[m][i] = ld_b128(x + (size_t)m * K, (uint32_t)min((int)threadIdx.x + i * threads, words - 1) * 16u);
    rw[m] = 0;
    if constexpr (kPro == kProPlain && kLW > 0) rw[m] = ld_b32(r + (size_t)m * rank, (uint32_t)min((int)threadIdx.x, ldw_half - 1) * 4u);
  }
  if constexpr (kPro == kProNormAcc) {
#pragma unroll
    for (int i = 0; i < kXW; ++i) nw[i] = ld_b128(ch.norm_w, (uint32_t)min((int)threadIdx.x + i * threads, words - 1) * 16u);
  }
  if constexpr (kAccPro) {
    // Loads and waits are unconditional (a copy past the last one is clamped to it and left out of the sum below): the
    // compiler takes the result of a load statement for present as soon as the statement has run, so a load under a
    // condition gets its result copied to the variable's register where the branches meet -- before the data is there
    // -- and the register the data then lands in is handed to something else.
#pragma unroll
    for (int a = 0; a < kAL; ++a) {
      const int c = min(wave + a * waves, kAccCopies - 1);
#pragma unroll
      for (int j = 0; j < kLW; ++j) av[a][j] = ld_b128(ch.acc_in + (size_t)c * kAccStride + 128 * j, (uint32_t)lane * 16u);
    }
  }

  // ---- member of this workgroup (one round trip to the argument buffer, overlapped with the loads above)
  MemberDev mem = g.mem[0];
  int wg_begin = 0, total_blocks = g.task_end[0];
  if constexpr (kEpi == kEpiNone) {
#define GLOWQ_PICK(i)                                            \
  if (g.n_members > i && wg >= g.wg_end[i - 1]) {               \
    mem = g.mem[i];                                              \
    wg_begin = g.wg_end[i - 1];                                  \
    total_blocks = g.task_end[i] - g.task_end[i - 1];            \
  }
    GLOWQ_PICK(1)
    GLOWQ_PICK(2)
    GLOWQ_PICK(3)
#undef GLOWQ_PICK
  }
  const int want = (wg - wg_begin) * waves + wave;
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
  // plain and residual forms: rows 2 blk and 2 blk + 1 of the member; gate/up pair: row blk of member 0 and of member 1
  Slot<kKit, kLW, kPacked, kEpi> b;
  const int n0 = kEpi == kEpiSwiglu ? blk : blk * kSRows;
  const bool two = kEpi == kEpiSwiglu ? true : n0 + 1 < mem.N;  // the second row exists
  {
    const char* w0 = reinterpret_cast<const char*>(mem.qweight + (size_t)n0 * mem.ldw);
    const char* w1 = two ? w0 + (size_t)mem.ldw * 4 : w0;
    if constexpr (kEpi == kEpiSwiglu) w1 = reinterpret_cast<const char*>(g.mem[1].qweight + (size_t)n0 * g.mem[1].ldw);
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
      if constexpr (kEpi == kEpiSwiglu) {
        // the upper half wave reads the row of the second member: an address per lane
        const char* sc1 = reinterpret_cast<const char*>(g.mem[1].scales + (size_t)n0 * g.mem[1].lds);
        const char* zw1 = reinterpret_cast<const char*>(g.mem[1].qzeros + (size_t)n0 * g.mem[1].ldz);
        const char* scl = rsel ? sc1 : sc0;
        const char* zwl = rsel ? zw1 : zw0;
#pragma unroll
        for (int p = 0; p < kNP; ++p) {
          b.sc[p] = ld_u16_nt_at(scl + ((sgrp[p] * 2u) & live));
          b.zw[p] = ld_b32_nt_at(zwl + (((sgrp[p] >> 3) * 4u) & live));
        }
      } else {
        const uint32_t sc_row = two ? (uint32_t)mem.lds * 2u : 0u, zw_row = two ? (uint32_t)mem.ldz * 4u : 0u;
#pragma unroll
        for (int p = 0; p < kNP; ++p) {
          b.sc[p] = ld_u16_nt(sc0, (rsel * sc_row + sgrp[p] * 2u) & live);
          b.zw[p] = ld_b32_nt(zw0, (rsel * zw_row + (sgrp[p] >> 3) * 4u) & live);
        }
      }
      if constexpr (kLW > 0) {
        // a member without L reads r itself (valid memory; x where r is produced inside the launch) and is weighted by zero
        const half_t* some = kPro == kProPlain ? r : kPro == kProProj ? x : reinterpret_cast<const half_t*>(ch.acc_in);
        const char* l0 = mem.L ? reinterpret_cast<const char*>(mem.L + (size_t)n0 * rank) : reinterpret_cast<const char*>(some);
        const char* l1 = (mem.L && two) ? l0 + (size_t)rank * 2 : l0;
        if constexpr (kEpi == kEpiSwiglu) l1 = reinterpret_cast<const char*>(g.mem[1].L + (size_t)n0 * rank);
#pragma unroll
        for (int j = 0; j < kLW; ++j) {
          const uint32_t lo = ((uint32_t)min(lane + kWave * j, ldw_half - 1) * 4u) & live;
          b.l[0][j] = ld_b32_nt(l0, lo);
          b.l[1][j] = ld_b32_nt(l1, lo);
        }
      }
    }
    if constexpr (kEpi != kEpiNone && kLW > 0) {
      // rows n0 (and n0 + 1) of the next group's transposed right factor; without one, any valid memory
      const char* t0 = ch.next_rt ? reinterpret_cast<const char*>(ch.next_rt + (size_t)n0 * rank) : reinterpret_cast<const char*>(x);
      const char* t1 = (ch.next_rt && two) ? t0 + (size_t)rank * 2 : t0;
#pragma unroll
      for (int j = 0; j < kLW; ++j) {
        const uint32_t lo = ((uint32_t)min(lane + kWave * j, ldw_half - 1) * 4u) & live;
        b.rt[0][j] = ld_b32_nt(t0, lo);
        if constexpr (kEpi == kEpiResidual) b.rt[1][j] = ld_b32_nt(t1, lo);
      }
    }
#pragma unroll
    for (int it = 0; it < kKit; ++it) {
      const uint32_t vo = it == kKit - 1 ? voff_last : voff;
      b.w[it][0] = ld_b128_nt(w0 + it * 1024, vo);
      b.w[it][1] = ld_b128_nt(w1 + it * 1024, vo);
    }
  }
  // the epilogue's scalars: requested here, needed after the last step
  float e_bias0 = 0.f, e_bias1 = 0.f, e_res0 = 0.f, e_res1 = 0.f, e_w0 = 1.f, e_w1 = 1.f;
  if constexpr (kEpi == kEpiResidual) {
    const int n1 = two ? n0 + 1 : n0;
    if (mem.bias) { e_bias0 = (float)mem.bias[n0]; e_bias1 = (float)mem.bias[n1]; }
    e_res0 = (float)ch.resid[n0];
    e_res1 = (float)ch.resid[n1];
    if (ch.next_w) { e_w0 = (float)ch.next_w[n0]; e_w1 = (float)ch.next_w[n1]; }
  }
  if constexpr (kEpi == kEpiSwiglu) {
    if (mem.bias) e_bias0 = (float)mem.bias[n0];
    if (g.mem[1].bias) e_bias1 = (float)g.mem[1].bias[n0];
  }

  // ---- stage the activations (every load of x and r lies ahead of the row block's: one count covers them all)
  float norm_f = 1.f;
  if constexpr (kPro == kProNormAcc) {
    // the norm factor first: sum of squares of the row over the workgroup (fp32, lanes, then waves in wave order)
    wait_words<C::kLoads>(xw[0]);
    wait_words<C::kLoads>(nw);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kXW; ++i) {
      if ((int)threadIdx.x + i * threads < words) {
        const h8 v = __builtin_bit_cast(h8, xw[0][i]);
#pragma unroll
        for (int e = 0; e < 8; e += 2) ss = __builtin_amdgcn_fdot2(h2{v[e], v[e + 1]}, h2{v[e], v[e + 1]}, ss, false);
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < waves; ++i) t += red[i];
    norm_f = rsqrtf(t / (float)K + ch.eps);
    // h = fp16(fp16(x f) w): the rounding steps of the norm kernel it replaces
#pragma unroll
    for (int i = 0; i < kXW; ++i) {
      const h8 v = __builtin_bit_cast(h8, xw[0][i]);
      const h8 wv = __builtin_bit_cast(h8, nw[i]);
      h8 o;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const h2 n2 = {(half_t)((float)v[e] * norm_f), (half_t)((float)v[e + 1] * norm_f)};
        const h2 o2 = n2 * h2{wv[e], wv[e + 1]};
        o[e] = o2[0];
        o[e + 1] = o2[1];
      }
      xw[0][i] = __builtin_bit_cast(u32x4, o);
    }
  }
#pragma unroll
  for (int m = 0; m < kM; ++m) {
    if constexpr (kPro != kProNormAcc) wait_words<C::kLoads>(xw[m]);
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
    if constexpr (kPro == kProPlain && kLW > 0) {
      wait_vm<C::kLoads>(rw[m]);
      if ((int)threadIdx.x < ldw_half) reinterpret_cast<uint32_t*>(rs + (size_t)m * rank)[threadIdx.x] = rw[m];
    }
  }
  if constexpr (kAccPro) {
    // this wave's share of the sum over the copies, entry by entry, for every wave to pick up behind the barrier
#pragma unroll
    for (int j = 0; j < kLW; ++j) {
      long long s0 = 0, s1 = 0;
#pragma unroll
      for (int a = 0; a < kAL; ++a) {
        wait_vm<C::kLoads>(av[a][j]);
        const bool mine = wave + a * waves < kAccCopies;
        const long long e0 = (long long)(((unsigned long long)av[a][j][1] << 32) | av[a][j][0]);
        const long long e1 = (long long)(((unsigned long long)av[a][j][3] << 32) | av[a][j][2]);
        s0 += mine ? e0 : 0;
        s1 += mine ? e1 : 0;
      }
      long long* dst = accp + ((size_t)wave * kLW + j) * 128 + 2 * lane;
      dst[0] = s0;
      dst[1] = s1;
    }
  }
  __syncthreads();
  if constexpr (kEpi == kEpiNone && kPro != kProProj) {
    if (!valid) return;  // (after the barrier; the loads still in flight land in registers nobody reads)
  }
  // kProProj: thread t's first look at entry t of r (rank <= 256 <= threads) goes out ahead of the wait for the last
  // step's weights: as late as it can without adding a round trip of its own behind them
  u32x2 look = {0u, 0u};
  // ---- consume the row block in the order it was requested
  float tot[kSRows][kM];
#pragma unroll
  for (int rr = 0; rr < kSRows; ++rr)
#pragma unroll
    for (int m = 0; m < kM; ++m) tot[rr][m] = 0.f;
  // the correction's share: [L] . [alpha r], r from LDS (or, in the accumulator forms, from the sums staged there)
  auto apply_left = [&]() {
#pragma unroll
    for (int j = 0; j < kLW; ++j) {
      const int idx = lane + kWave * j;
      // (gate/up pair: both members carry L, checked on the host)
      const float a = idx < ldw_half ? alpha_scaled : 0.f;
#pragma unroll
      for (int m = 0; m < kM; ++m) {
        h2 rv;
        if constexpr (!kAccPro) {
          rv = reinterpret_cast<const h2*>(rs + (size_t)m * rank)[min(idx, ldw_half - 1)];
        } else {
          // r = fp16(f P), P = 2^-32 * (sum over the waves' shares); an accumulator that overflowed gives NaN
          const int li = min(idx, ldw_half - 1);
          long long s0 = 0, s1 = 0;
          for (int w = 0; w < waves; ++w) {
            const long long* src = accp + ((size_t)w * kLW + (li >> 6)) * 128 + 2 * (li & 63);
            s0 += src[0];
            s1 += src[1];
          }
          const float bad = ch.acc_in[(size_t)kAccCopies * kAccStride] != 0 ? __builtin_nanf("") : 0.f;
          rv = h2{(half_t)((float)s0 * 0x1p-32f * norm_f + bad), (half_t)((float)s1 * 0x1p-32f * norm_f + bad)};
        }
#pragma unroll
        for (int rr = 0; rr < kSRows; ++rr)
          tot[rr][m] = __builtin_fmaf(a, __builtin_amdgcn_fdot2(bitcast_u32<h2>(kPacked ? b.side(kNP + kSRows * j + rr) : b.l[rr][j]),
                                                             rv, 0.f, false), tot[rr][m]);
      }
    }
  };
  float held_sc[kPro == kProProj ? kKit : 1][kSRows], held_v[kPro == kProProj ? kKit : 1][kSRows];
  uint32_t rec = 0;
  static_for<kKit>([&](auto IT) {
    constexpr int it = decltype(IT)::value;
    constexpr int p = it >> 1;
    constexpr int kBehind = kSRows * (kKit - 1 - it) + (it == kKit - 1 ? kLook : 0);  // loads issued behind the weights of this step
    if constexpr (kPro == kProProj && it == kKit - 1) look = ld_b64_agent(ch.proj_pub, (uint32_t)min((int)threadIdx.x, rank - 1) * 8u);
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
      if constexpr (kEpi != kEpiNone) {
#pragma unroll
        for (int j = 0; j < kLW; ++j) {
          wait_vm<kBehind>(b.rt[0][j]);
          if constexpr (kEpi == kEpiResidual) wait_vm<kBehind>(b.rt[1][j]);
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
        if constexpr (kPro == kProProj && it > 0) {
          // held back: the sums of every form add in the same order (step 0, the correction, the other steps), and here
          // the correction has to wait for r
          held_sc[it][rr] = sc[rr];
          held_v[it][rr] = v;
        } else {
          tot[rr][m] = __builtin_fmaf(sc[rr], v, tot[rr][m]);
        }
      }
    }
    if constexpr (it == 0 && kLW > 0 && kPro != kProProj) apply_left();
    // The step's sums are pinned here (an empty statement that "rewrites" them): left alone, the compiler sinks the whole
    // arithmetic of every step to the point of the reduction below, behind all the waits, and keeps every loaded word
    // and activation fragment of every step live until then (30 VGPRs per step and token row).
#pragma unroll
    for (int rr = 0; rr < kSRows; ++rr) {
#pragma unroll
      for (int m = 0; m < kM; ++m) asm volatile("" : "+v"(tot[rr][m]));
      if constexpr (kPro == kProProj && it > 0) asm volatile("" : "+v"(held_v[it][rr]));
    }
  });
  if constexpr (kPro == kProProj) {
    // r from the waves that produced it: thread t has looked at entry t; where the word was not there yet it looks again
    wait_vm<0>(look);
    if ((int)threadIdx.x < rank) {
      unsigned long long w = ((unsigned long long)look[1] << 32) | look[0];
      unsigned spins = 0;
      bool seen = (w & kTagMask) == tag;
      while (!seen && spins < ch.proj_spin) {
        ++spins;
        w = __hip_atomic_load(ch.proj_pub + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        seen = (w & kTagMask) == tag;
        if (!seen) __builtin_amdgcn_s_sleep(2);
      }
      half_t v = __builtin_bit_cast(half_t, (uint16_t)(w >> 48));
      if (!seen) {
        // the producer has not been heard from within the limit: this thread's own dot product (fp32, column order)
        const half_t* Rrow = ch.proj_R + (size_t)threadIdx.x * K;
        float acc = 0.f;
        for (int k = 0; k < K; ++k) acc = __builtin_fmaf((float)Rrow[k], (float)x[k], acc);
        v = (half_t)acc;
      }
      rs[threadIdx.x] = v;
    }
    __syncthreads();
    apply_left();
#pragma unroll
    for (int it = 1; it < kKit; ++it)
#pragma unroll
      for (int rr = 0; rr < kSRows; ++rr) tot[rr][0] = __builtin_fmaf(held_sc[it][rr], held_v[it][rr], tot[rr][0]);
  }
  // lane rr keeps the total of row rr: one store (and one bias load) per token row
  const int n = blk * kSRows + lane;
  const bool writer = valid && lane < kSRows && n < mem.N;
  float bias = 0.f;
  if constexpr (kEpi == kEpiNone) bias = (writer && mem.bias) ? (float)mem.bias[n] : 0.f;
  float row0 = 0.f, row1 = 0.f;
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
    row0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    row1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    if constexpr (kEpi == kEpiNone) {
      const float mine = lane == 0 ? row0 : row1;
      if (writer) mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(mine, 0x1p24f, bias));
    }
  }

  // ---- chained epilogues (row0 and row1 are the same in every lane)
  if constexpr (kEpi != kEpiNone) {
    float c0 = 0.f, c1 = 0.f;  // what the wave's rows contribute to the next projection
    if constexpr (kEpi == kEpiResidual) {
      const half_t y0 = (half_t)__builtin_fmaf(row0, 0x1p24f, e_bias0), y1 = (half_t)__builtin_fmaf(row1, 0x1p24f, e_bias1);
      const half_t x0 = (half_t)(e_res0 + (float)y0), x1 = (half_t)(e_res1 + (float)y1);
      if (valid && lane == 0) {
        ch.resid[n0] = x0;
        if (mem.y) mem.y[n0] = y0;
      }
      if (valid && two && lane == 1) {
        ch.resid[n0 + 1] = x1;
        if (mem.y) mem.y[n0 + 1] = y1;
      }
      c0 = valid ? e_w0 * (float)x0 : 0.f;
      c1 = (valid && two) ? e_w1 * (float)x1 : 0.f;
    } else {
      const half_t gt = (half_t)__builtin_fmaf(row0, 0x1p24f, e_bias0), up = (half_t)__builtin_fmaf(row1, 0x1p24f, e_bias1);
      const half_t a = (half_t)((float)(half_t)silu_f32((float)gt) * (float)up);
      if (valid && lane == 0) {
        ch.act[n0] = a;
        if (mem.y) mem.y[n0] = gt;
        if (g.mem[1].y) g.mem[1].y[n0] = up;
      }
      c0 = valid ? (float)a : 0.f;
    }
    if constexpr (kLW > 0) {
      if (ch.next_rt != nullptr) {
#pragma unroll
        for (int j = 0; j < kLW; ++j) {
          const int idx = lane + kWave * j;
          if (idx < ldw_half) {
            const h2 t0 = bitcast_u32<h2>(b.rt[0][j]);
            float p0 = c0 * (float)t0[0], p1 = c0 * (float)t0[1];
            if constexpr (kEpi == kEpiResidual) {
              const h2 t1 = bitcast_u32<h2>(b.rt[1][j]);
              p0 = __builtin_fmaf(c1, (float)t1[0], p0);
              p1 = __builtin_fmaf(c1, (float)t1[1], p1);
            }
            part[wave * rank + 2 * idx] = p0;
            part[wave * rank + 2 * idx + 1] = p1;
          }
        }
        __syncthreads();
        if ((int)threadIdx.x < rank) {
          float s = 0.f;
          for (int w = 0; w < waves; ++w) s += part[w * rank + threadIdx.x];
          unsigned long long* slot = reinterpret_cast<unsigned long long*>(ch.acc_out) + (size_t)(blockIdx.x & (kAccCopies - 1)) * kAccStride;
          if (fabsf(s) < ch.part_limit) atomicAdd(slot + threadIdx.x, (unsigned long long)__float2ll_rn(s * 0x1p32f));
          else ch.acc_out[(size_t)kAccCopies * kAccStride] = 1;  // too large for the fixed point, or NaN
        }
      }
    }
  }
}

}  // namespace streamk
}  // namespace glowq
