// Skinny MFMA route for a handful of token rows (5 <= M <= 64): the weights are streamed once, like in the
// GEMV, but the multiply-accumulate work goes to the matrix cores.
//
// A workgroup owns 32*kNT output columns of one member and all M rows; its waves split K: wave w takes the
// a contiguous range of 64-deep blocks and keeps a private 32*kMT x 32*kNT accumulator tile
// (v_mfma_f32_32x32x16_f16).  Nothing is shared between the waves while they stream, so there is no
// barrier in the loop and every wave runs its own three-deep prefetch:
//   * B operand: one 16-byte load of int4 codes per lane, block and column tile, dequantised in registers to
//     fp16((code - zero) * scale) exactly as in the tiled GEMM;
//   * A operand: the lane's 8 activations per MFMA step straight from global memory (x is a few hundred KB at
//     most and lives in L2), permuted in registers into the order the nibble masks deliver the codes.  With
//     kNT >= 2 every A fragment feeds two MFMAs, which keeps the L1 traffic per weight byte low enough.
// The correction is a K-extension in front: the ceil(rank/64) blocks of [r | L] are dealt to the waves first,
// acc *= alpha, then the weight blocks accumulate on top.  The waves' partial tiles meet in LDS once.  (Where the launch
// computes r itself -- the second form's kProj -- the correction comes behind the weights instead.)
#include <atomic>
#include <cstdlib>

#include "common.hpp"
#include "handover.hpp"
#include "proj_block.hpp"

namespace glowq {

struct SkinnyMember {
  const int32_t* qweight;
  const half_t* scales;
  const int32_t* qzeros;
  const half_t* L;
  const half_t* bias;
  half_t* y;
  int N, ldw, lds, ldz, ldy;
};

struct SkinnyArgs {
  const half_t* x;  // [M, K]
  const half_t* r;  // [M, rank] or nullptr
  SkinnyMember mem[GLOWQ_MAX_MEMBERS];
  int blk_end[GLOWQ_MAX_MEMBERS];
  int n_members;
  int M, K, rank, gs_shift;
  float alpha;
  // second form only: gridDim.y slices of whole super-blocks; with more than one, every workgroup leaves its fp32
  // tile in `partials` ([slice][workgroup][M][32 kNT]) and skinny_reduce_kernel adds the slices in order
  int slices;
  float* partials;
  // second form, where the launch computes r = x R^T itself (kProj): workgroups in front of the grid produce blocks of
  // four token rows by four rows of R and write them to r_out, the others apply the correction behind their weights
  // instead of in front of them and read r_out once the word `pub[0]` says that all of it is there
  const half_t* R;          // [rank, K]
  half_t* r_out;            // [M, rank]
  unsigned long long* pub;  // [0]: the ready word; [kSkinnyFlags + p]: the flag of producer p
  unsigned spin;            // polls of the ready word before a wave computes its part of r itself
  int producers;            // workgroups that produce r
  int teams;                // blocks of r a producer works on at a time: teams of four waves (1 or 2)
};
constexpr int kSkinnyFlags = 512;          // the producers' flags lie 4096 bytes behind the ready word
constexpr int kSkinnyMaxProducers = 512;
constexpr size_t kSkinnyHandoverBytes = (size_t)(kSkinnyFlags + kSkinnyMaxProducers) * 8;

__device__ __forceinline__ h8 nibble_order(const u32x4& v) {
  // halves (0..7) -> (0,4,1,5,2,6,3,7): two byte permutes per output dword
  u32x4 o;
  o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (h0, h4)
  o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (h1, h5)
  o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (h2, h6)
  o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (h3, h7)
  return __builtin_bit_cast(h8, o);
}

// total over a row of 16 lanes, in every lane of it
__device__ __forceinline__ float row16_total(float v) {
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xF, 0xF, true);  // row_ror:1
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xF, 0xF, true);  // row_ror:2
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true);  // row_ror:4
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true);  // row_ror:8
  v += __builtin_bit_cast(float, t);
  return v;
}

__device__ __forceinline__ h8 dequant_word_sk(uint32_t w, h2 zb_lo, h2 zb_hi, h2 s2) {
  // the two exponent patterns (1024.0 and 64.0 in both halves) are held in vector registers: with the nibble mask as
  // the one scalar operand each mask-and-merge is a single v_and_or_b32 instead of an AND and an OR
  uint32_t e1024, e64;
  asm("v_mov_b32 %0, 0x64006400" : "=v"(e1024));
  asm("v_mov_b32 %0, 0x54005400" : "=v"(e64));
  const uint32_t hi = w >> 8;
  const h2 q0 = bitcast_u32<h2>((w & 0x000F000Fu) | e1024);
  const h2 q1 = bitcast_u32<h2>((w & 0x00F000F0u) | e64);
  const h2 q2 = bitcast_u32<h2>((hi & 0x000F000Fu) | e1024);
  const h2 q3 = bitcast_u32<h2>((hi & 0x00F000F0u) | e64);
  const h2 d0 = (q0 + zb_lo) * s2;
  const h2 d1 = (q1 + zb_hi) * s2;
  const h2 d2 = (q2 + zb_lo) * s2;
  const h2 d3 = (q3 + zb_hi) * s2;
  h8 out;
  out[0] = d0[0]; out[1] = d0[1]; out[2] = d1[0]; out[3] = d1[1];
  out[4] = d2[0]; out[5] = d2[1]; out[6] = d3[0]; out[7] = d3[1];
  return out;
}

// What one block needs: per column tile 16 bytes of codes (or 4 x 16 bytes of L), scale and zero-point word,
// and per row tile the four A fragments.
template <int kMT, int kNT>
struct SkinnyRegs {
  u32x4 a[kMT][4];
  u32x4 b[kNT];
  uint32_t s[kNT];
  uint32_t z[kNT];
};

template <int kMT, int kNT>
__global__ __launch_bounds__(512) void skinny_mfma_kernel(const SkinnyArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int ln = lane & 31, lh = lane >> 5;

  SkinnyMember mem = g.mem[0];
  int blk_base = 0;
#define GLOWQ_PICK(i)                                          \
  if (g.n_members > i && (int)blockIdx.x >= g.blk_end[i - 1]) { \
    mem = g.mem[i];                                            \
    blk_base = g.blk_end[i - 1];                               \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int n0 = ((int)blockIdx.x - blk_base) * (32 * kNT);

  int ncol[kNT];
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) ncol[tn] = min(n0 + tn * 32 + ln, mem.N - 1);
  int mrow[kMT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm) mrow[tm] = min(tm * 32 + ln, g.M - 1);

  f16v acc[kMT][kNT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tm][tn][i] = 0.f;

  // ---- phase 1: correction blocks [r | L], fp16 B operand, dealt round-robin to the waves ----------------
  const bool corrected = mem.L != nullptr && g.r != nullptr;
  if (corrected) {
    const int lblocks = (g.rank + 63) >> 6;  // ranks are multiples of 8: the last block may be partial
    for (int jb = wave; jb < lblocks; jb += waves) {
      const int kb = jb * 64;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // octets past the rank: r counts as zero there, L is read from the row's last octet (finite values)
        const int k = kb + 32 * lh + 8 * t;
        const bool live = k < g.rank;
        const int kc = min(k, g.rank - 8);
        h8 af[kMT];
#pragma unroll
        for (int tm = 0; tm < kMT; ++tm)
          af[tm] = live ? *reinterpret_cast<const h8*>(g.r + (size_t)mrow[tm] * g.rank + kc) : h8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) {
          const h8 bf = *reinterpret_cast<const h8*>(mem.L + (size_t)ncol[tn] * g.rank + kc);
#pragma unroll
          for (int tm = 0; tm < kMT; ++tm) acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tm], bf, acc[tm][tn], 0, 0, 0);
        }
      }
    }
    if (g.alpha != 1.0f) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[tm][tn][i] *= g.alpha;
    }
  }

  // ---- phase 2: weight blocks, three register sets in rotation ------------------------------------------
  // Wave w walks the contiguous block range [w*per, (w+1)*per): consecutive steps of a wave touch
  // consecutive 32-byte pieces of the same 128-byte lines of its 32 weight rows, so every line is fetched
  // from HBM once and re-used out of L2.
  const int kblocks = g.K >> 6;
  const int per = (kblocks + waves - 1) / waves;
  const int first_blk = wave * per;
  const int my_blocks = max(0, min(per, kblocks - first_blk));
  auto issue = [&](int i, SkinnyRegs<kMT, kNT>& rg) {
    const int blk = min(first_blk + i, kblocks - 1);  // past-the-end prefetches re-read the last block
    const int kb = blk * 64;
    const int grp = (kb + 32 * lh) >> g.gs_shift;
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      rg.b[tn] = *reinterpret_cast<const u32x4*>(mem.qweight + (size_t)ncol[tn] * mem.ldw + (kb >> 3) + 4 * lh);
      rg.s[tn] = reinterpret_cast<const unsigned short*>(mem.scales)[(size_t)ncol[tn] * mem.lds + grp];
      rg.z[tn] = (uint32_t)mem.qzeros[(size_t)ncol[tn] * mem.ldz + (grp >> 3)];
    }
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        rg.a[tm][t] = *reinterpret_cast<const u32x4*>(g.x + (size_t)mrow[tm] * g.K + kb + 32 * lh + 8 * t);
  };
  auto compute = [&](int i, const SkinnyRegs<kMT, kNT>& rg) {
    const int kb = (first_blk + i) * 64;
    const int grp = (kb + 32 * lh) >> g.gs_shift;
    h8 bf[kNT][4];
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      const half_t z = (half_t)(float)nibble(rg.z[tn], grp & 7);
      const half_t zl = (half_t)(-1024.0f) - z, zh = (half_t)(-64.0f) - z;
      const h2 zb_lo = {zl, zl}, zb_hi = {zh, zh};
      const h2 s2 = bitcast_u32<h2>(rg.s[tn] | (rg.s[tn] << 16));
      bf[tn][0] = dequant_word_sk(rg.b[tn].x, zb_lo, zb_hi, s2);
      bf[tn][1] = dequant_word_sk(rg.b[tn].y, zb_lo, zb_hi, s2);
      bf[tn][2] = dequant_word_sk(rg.b[tn].z, zb_lo, zb_hi, s2);
      bf[tn][3] = dequant_word_sk(rg.b[tn].w, zb_lo, zb_hi, s2);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm) {
        const h8 af = nibble_order(rg.a[tm][t]);
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf[tn][t], acc[tm][tn], 0, 0, 0);
      }
    }
  };

  // The fences pin the loads where they are written: with no barrier in this loop the compiler is otherwise
  // free to sink them down to their uses, which would collapse the three-deep pipeline into none.
#define GLOWQ_PIN_LOADS() asm volatile("" ::: "memory")
  SkinnyRegs<kMT, kNT> r0, r1, r2;
  issue(0, r0);
  issue(1, r1);
  GLOWQ_PIN_LOADS();
  for (int i = 0; i < my_blocks; i += 3) {
    issue(i + 2, r2);
    GLOWQ_PIN_LOADS();
    compute(i, r0);
    if (i + 1 >= my_blocks) break;
    issue(i + 3, r0);
    GLOWQ_PIN_LOADS();
    compute(i + 1, r1);
    if (i + 2 >= my_blocks) break;
    issue(i + 4, r1);
    GLOWQ_PIN_LOADS();
    compute(i + 2, r2);
  }
#undef GLOWQ_PIN_LOADS

  // ---- the waves' partial tiles meet in LDS: [wave][tm][tn][16 regs][64 lanes] floats, in rounds of 8 waves
  float* red = reinterpret_cast<float*>(smem);
  constexpr int kTile = kMT * kNT * 16 * 64;
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
      for (int i = 0; i < 16; ++i) red[(size_t)wave * kTile + ((tm * kNT + tn) * 16 + i) * 64 + lane] = acc[tm][tn][i];
  __syncthreads();
  // every thread finishes a share of the (tile, register, lane) slots
  const int slots = kMT * kNT * 16 * 64;
  for (int sidx = threadIdx.x; sidx < slots; sidx += blockDim.x) {
    float v = 0.f;
    for (int w = 0; w < waves; ++w) v += red[(size_t)w * kTile + sidx];
    const int l = sidx & 63;
    const int i = (sidx >> 6) & 15;
    const int tt = sidx >> 10;
    const int tm = tt / kNT, tn = tt - tm * kNT;
    const int n = n0 + tn * 32 + (l & 31);
    const int m = tm * 32 + 8 * (i >> 2) + 4 * (l >> 5) + (i & 3);
    if (m < g.M && n < mem.N) {
      const float b = mem.bias ? (float)mem.bias[n] : 0.f;
      mem.y[(size_t)m * mem.ldy + n] = (half_t)(v + b);
    }
  }
}

// Second form of the kernel for K % 256 == 0 and group sizes of 128 and up.  A wave walks 256-deep super-blocks;
// lane (column c, half h) owns the 64 contiguous bytes of row c that hold codes [256 sb + 128 h, +128): exactly one
// quantisation group, so one scale and one zero-point per lane, column tile and super-block, and the four 16-byte loads
// of a lane hit the same 128-byte line back to back (the first form touches every line in four separate blocks and
// fetches scale and zero-point with every one of them).  The activations follow the same k assignment, but reach the
// A operand through a wave-private LDS tile: the wave loads the 128-byte row segments of half a super-block in memory
// order (8 lanes per segment, every line requested once per instruction) and reads the fragments back in MFMA lane
// order.  Loading the fragments straight from memory (one 16-byte request per lane and line) cost 22 us of the 45 us
// of a 28672 x 4096 layer at 32 rows: every request pulls a whole line out of L2.
// kRaw (groups of 128 columns): the codes go to the matrix cores as they are -- masked in place they are the fp16
// subnormals code * 2^-24 and code * 2^-20, the activations of the latter staged divided by 16 -- with all sixteen k
// values of an instruction inside one group: lane (column c, half h) takes the 32-column quarters h and 2 + h of the
// group instead of one whole group of the super-block.  The eight instructions of a group leave its plain sum of
// code * x, and scale and zero-point are applied to that sum, y += s (sum c x - z sum x), with the fp32 sums of x per
// token row and group taken when the activations are staged.  Five vector instructions per code word instead of
// thirteen, and the arithmetic of the GEMV routes: weights never rounded to fp16.
// kProj: the launch computes r = x R^T itself (SkinnyArgs).  The grid then has `producers` workgroups in front (roles
// dealt as in handover.hpp).  A producer's teams of four waves (one or two) each take every (producers x teams)-th block of
// four token rows by four rows of R, in the arithmetic of shared_proj_block_kernel; the producer writes them to r_out with
// stores that pass the caches private to a part of the chip, waits until they are acknowledged and raises its flag (the
// launch's tag); the first producer then polls all flags (bounded) and, when all are up, writes the ready word.  A wave with a correction block polls the ready word (bounded)
// once its weights are done, then reads its part of r with loads that pass those caches as well; a wave that never sees
// the word computes the part of r it needs itself, so every wave ends whatever becomes of the producers.
template <int kMT, int kNT, bool kBulk, bool kRaw, bool kProj = false>
__global__ __launch_bounds__(512) void skinny_group_kernel(const SkinnyArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int ln = lane & 31, lh = lane >> 5;

  int wg = (int)blockIdx.x;
  const int tiles = g.blk_end[g.n_members - 1];  // workgroups with a column tile (per slice)
  unsigned long long tag = 0;
  if constexpr (kProj) {
    tag = launch_tag();
    const int front = g.producers;
    const int role = front_role(wg, front);
    if (role >= 0) {
      if (role >= front || blockIdx.y != 0) return;
      {
        // teams of 256 threads, each with a block of its own at a time: two where the workgroup has eight waves (the
        // round trips of two blocks overlap; the compute unit has nothing else to do)
        const int teams = g.teams;
        if ((int)threadIdx.x >= 256 * teams) return;  // (the body's barriers count the waves that arrive)
        const int team = (int)threadIdx.x >> 8, tid = (int)threadIdx.x & 255;
        float* part = reinterpret_cast<float*>(smem) + team * (4 * 16 + 16);
        float* vals = part + 4 * 16;
        const int jblocks = (g.rank + 3) >> 2, nblocks = jblocks * ((g.M + 3) >> 2);
        // blocks of four token rows by four rows of R, dealt round robin to the teams of the producers
        for (int b0 = role * teams; b0 < nblocks; b0 += g.producers * teams) {
          const int b = b0 + team;
          const bool active = b < nblocks;
          const int bj = b % jblocks, bm = b / jblocks;
          proj_block_body<4, 4>(g.x, g.R, g.M, g.K, g.rank, 4 * bj, 4 * bm, part,
                                [&](int m, int j, float v) { vals[(m - 4 * bm) * 4 + (j - 4 * bj)] = v; }, tid, active);
          __syncthreads();
          // pairs of neighbouring entries of a token row go out as one 32-bit store (ranks are multiples of 8)
          if (active && tid < 8) {
            const int mi = tid >> 1, pp = tid & 1;
            const int m = 4 * bm + mi, j = 4 * bj + 2 * pp;
            if (m < g.M && j < g.rank) {
              const h2 v = {(half_t)vals[mi * 4 + 2 * pp], (half_t)vals[mi * 4 + 2 * pp + 1]};
              __hip_atomic_store(reinterpret_cast<uint32_t*>(g.r_out + (size_t)m * g.rank + j), __builtin_bit_cast(uint32_t, v),
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          }
          __syncthreads();  // (part and vals are free for the next block)
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores are acknowledged: r is where every reader looks
        __syncthreads();
        if (threadIdx.x == 0 && g.spin != 0xFFFFFFFFu)  // (that value: a test in which the flags never go up)
          __hip_atomic_store(g.pub + kSkinnyFlags + role, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      // the first producer is also the collector: one wave, lane l takes flags l, l + 64, ...  (a workgroup of its own
      // for this takes a place that a producer can use: 64 blocks of r for 64 free compute units)
      if (role != 0 || wave != 0) return;
      bool all = false;
      for (unsigned spins = 0; !all && spins <= g.spin && g.spin != 0xFFFFFFFFu; ++spins) {
        bool mine = true;
        for (int p = lane; p < g.producers; p += 64)
          mine = mine && (__hip_atomic_load(g.pub + kSkinnyFlags + p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & kTagMask) == tag;
        all = __builtin_amdgcn_ballot_w64(!mine) == 0;
        if (!all) __builtin_amdgcn_s_sleep(2);
      }
      if (all && lane == 0) __hip_atomic_store(g.pub, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (wg >= tiles) return;  // (a front larger than the grid behind it leaves places between its workgroups empty)
  }

  SkinnyMember mem = g.mem[0];
  int blk_base = 0;
#define GLOWQ_PICK(i)                                          \
  if (g.n_members > i && wg >= g.blk_end[i - 1]) {             \
    mem = g.mem[i];                                            \
    blk_base = g.blk_end[i - 1];                               \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int n0 = (wg - blk_base) * (32 * kNT);

  int ncol[kNT];
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) ncol[tn] = min(n0 + tn * 32 + ln, mem.N - 1);
  int mrow[kMT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm) mrow[tm] = min(tm * 32 + ln, g.M - 1);

  f16v acc[kMT][kNT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tm][tn][i] = 0.f;

  // ---- phase 1: correction blocks [r | L], fp16 B operand, dealt round-robin to the waves ----------------
  constexpr int kSegStride = 144;                      // 128 bytes of a row segment + 16: conflict-free fragment reads
  constexpr int kATile = kMT * 64 * kSegStride;        // bytes per wave
  constexpr int kBTile = kNT * 32 * kSegStride;
  constexpr int kSig = kRaw ? kMT * 32 * (int)sizeof(float) : 0;  // sums of x over the group being staged, per token row
  unsigned char* atile = smem + (size_t)wave * (kATile + kBTile + kSig);
  unsigned char* btile = atile + kATile;
  float* asig = reinterpret_cast<float*>(btile + kBTile);
  const bool corrected = mem.L != nullptr && (kProj || g.r != nullptr) && blockIdx.y == 0;  // the first slice carries the correction
  const int lblocks = (g.rank + 63) >> 6;  // ranks are multiples of 8: the last block may be partial
  // A 64-column block of [r | L] reaches the operands like the weights below: its 128-byte row segments are loaded in
  // memory order, 8 lanes per segment, into the wave's LDS tiles and read back in MFMA lane order.
  // r_there (kProj): r_out holds r; else the lane computes the octets of r it would have loaded (fp32, column order).
  auto correction = [&](const bool r_there) {
    for (int jb = wave; jb < lblocks; jb += waves) {
      // octets past the rank: r counts as zero there, L is read from the row's last octet (finite values)
      const int k = jb * 64 + (lane & 7) * 8;
      const bool live = k < g.rank;
      const int kc = min(k, g.rank - 8);
      u32x4 lreg[kNT * 4], rreg[kMT * 4];
#pragma unroll
      for (int q = 0; q < kMT * 4; ++q) {
        const int m = min(q * 8 + (lane >> 3), g.M - 1);
        if constexpr (kProj) {
          if (r_there) {
            // (64-bit loads of agent scope: they pass the caches that the producers' stores passed)
            const unsigned long long* src = reinterpret_cast<const unsigned long long*>(g.r_out + (size_t)m * g.rank + kc);
            const unsigned long long lo = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned long long hi = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            rreg[q] = u32x4{(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
          } else {
            h8 own;
            for (int e = 0; e < 8; ++e) {
              const half_t* Rrow = g.R + (size_t)(kc + e) * g.K;
              const half_t* xrow = g.x + (size_t)m * g.K;
              float a = 0.f;
              for (int kk = 0; kk < g.K; ++kk) a = __builtin_fmaf((float)Rrow[kk], (float)xrow[kk], a);
              own[e] = (half_t)a;
            }
            rreg[q] = __builtin_bit_cast(u32x4, own);
          }
        } else {
          rreg[q] = *reinterpret_cast<const u32x4*>(g.r + (size_t)m * g.rank + kc);
        }
        if (!live) rreg[q] = u32x4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int q = 0; q < kNT * 4; ++q)
        lreg[q] = *reinterpret_cast<const u32x4*>(mem.L + (size_t)min(n0 + q * 8 + (lane >> 3), mem.N - 1) * g.rank + kc);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous block are done
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < kMT * 4; ++q)
        *reinterpret_cast<u32x4*>(atile + (q * 8 + (lane >> 3)) * kSegStride + (lane & 7) * 16) = rreg[q];
#pragma unroll
      for (int q = 0; q < kNT * 4; ++q)
        *reinterpret_cast<u32x4*>(btile + (q * 8 + (lane >> 3)) * kSegStride + (lane & 7) * 16) = lreg[q];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        h8 af[kMT];
#pragma unroll
        for (int tm = 0; tm < kMT; ++tm)
          af[tm] = *reinterpret_cast<const h8*>(atile + (tm * 32 + ln) * kSegStride + lh * 64 + t * 16);
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) {
          const h8 bf = *reinterpret_cast<const h8*>(btile + (tn * 32 + ln) * kSegStride + lh * 64 + t * 16);
#pragma unroll
          for (int tm = 0; tm < kMT; ++tm) acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tm], bf, acc[tm][tn], 0, 0, 0);
        }
      }
    }
  };
  const auto scale_acc = [&](const float f) {
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tm][tn][i] *= f;
  };
  if constexpr (!kProj) {
    if (corrected) {
      correction(true);
      if (g.alpha != 1.0f) scale_acc(g.alpha);
    }
  }

  // ---- phase 2: super-blocks of 256 columns, contiguous range per wave ---------------------------------------
  struct BRegs {
    u32x4 b[kNT * 4];  // a super-block in load order: row 8 q + lane / 8 of the column tile, piece lane % 8
    uint32_t s[kNT], z[kNT];
  };
  struct ARegs {
    u32x4 a[kMT * 8];  // half a super-block in load order: segment 8 q + lane / 8, piece lane % 8
  };
  const int sblocks = g.K >> 8;
  // this workgroup's super-blocks: all of them, or slice blockIdx.y of g.slices; its waves split that range
  const int sb_slice = (sblocks + g.slices - 1) / g.slices;
  const int sb_begin = min((int)blockIdx.y * sb_slice, sblocks), sb_end = min(sb_begin + sb_slice, sblocks);
  const int per = (sb_end - sb_begin + waves - 1) / waves;
  const int first = sb_begin + wave * per;
  const int mine = max(0, min(per, sb_end - first));
  uint32_t cur_s[kNT], cur_z[kNT];  // scale bits and zero-point of the super-block being computed (kRaw: of both its
                                    // groups: two halves, two nibbles)

  // With groups of 128 columns a lane's scales and zero-points of eight consecutive super-blocks are 32 and 8
  // contiguous bytes of its weight row: they are fetched once per eight super-blocks (runs counted from the wave's
  // first super-block; one that would pass the end of the row is moved back to end with it) and kept in registers,
  // the lane's own half of every super-block picked out.  One scattered 2-byte and one 4-byte request per
  // super-block otherwise cost as much address processing as the super-block's weights.
  // The host picks this form (kBulk) where it applies; with five requests per run it is not worth it for waves with
  // fewer than four super-blocks.
  constexpr bool bulk = kBulk;
  u32x4 run_s[kNT];     // own scale of super-block j of the run: half j % 2 of dword j / 2
  u32x4 run_s2[kRaw ? kNT : 1];  // kRaw: run_s, run_s2 = the sixteen scales as loaded, dword j = both groups of super-block j
  uint64_t run_z[kNT];  // own zero-point of super-block j: byte j (kRaw: both groups' nibbles)
  int run_start = 0;    // first super-block of the run held
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) {
    run_s[tn] = u32x4{0u, 0u, 0u, 0u};
    run_z[tn] = 0;
  }
  auto fetch_run = [&](int start) {
    run_start = start;
    const int zword = start >> 2, zlast = (2 * sblocks - 1) >> 3;  // sixteen groups from group 2 start: two or three words
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      const uint32_t* srow = reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned short*>(mem.scales) + (size_t)ncol[tn] * mem.lds) + start;
      const u32x4 s0 = *reinterpret_cast<const u32x4*>(srow), s1 = *reinterpret_cast<const u32x4*>(srow + 4);
      const int32_t* zrow = mem.qzeros + (size_t)ncol[tn] * mem.ldz;
      const uint32_t z0 = (uint32_t)zrow[zword], z1 = (uint32_t)zrow[min(zword + 1, zlast)], z2 = (uint32_t)zrow[min(zword + 2, zlast)];
      if constexpr (kRaw) {
        run_s[tn] = s0;
        run_s2[tn] = s1;
        const int sh = 4 * ((2 * start) & 7);  // nibble of group 2 start
        const uint64_t lo = ((uint64_t)z1 << 32) | z0;
        run_z[tn] = sh ? (lo >> sh) | ((uint64_t)z2 << (64 - sh)) : lo;  // groups 2 start + 0..15, a nibble each
      } else {
      const uint32_t sel = lh ? 0x07060302u : 0x05040100u;  // upper or lower half of both dwords
      run_s[tn] = u32x4{__builtin_amdgcn_perm(s0.y, s0.x, sel), __builtin_amdgcn_perm(s0.w, s0.z, sel),
                        __builtin_amdgcn_perm(s1.y, s1.x, sel), __builtin_amdgcn_perm(s1.w, s1.z, sel)};
      const int sh = 4 * ((2 * start) & 7) + 4 * lh;  // nibble of group 2 start + lh
      const uint64_t lo = ((uint64_t)z1 << 32) | z0;
      const uint64_t a = sh ? (lo >> sh) | ((uint64_t)z2 << (64 - sh)) : lo;  // groups 2 start + lh + 0..15, a nibble each
      run_z[tn] = a & 0x0F0F0F0F0F0F0F0Full;
      }
    }
  };
  auto issue_b = [&](int i, BRegs& rb) {
    const int sb = min(first + i, sblocks - 1);  // past-the-end prefetches re-read the last one
    const int grp = (sb * 256 + lh * 128) >> g.gs_shift;
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = min(n0 + tn * 32 + q * 8 + (lane >> 3), mem.N - 1);
        rb.b[tn * 4 + q] = *reinterpret_cast<const u32x4*>(mem.qweight + (size_t)n * mem.ldw + sb * 32 + (lane & 7) * 4);
      }
      if (!bulk) {
        if constexpr (kRaw)  // both scales of the super-block (scale rows start on a 4-byte boundary: checked on the host)
          rb.s[tn] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned short*>(mem.scales) + (size_t)ncol[tn] * mem.lds + 2 * sb);
        else
          rb.s[tn] = reinterpret_cast<const unsigned short*>(mem.scales)[(size_t)ncol[tn] * mem.lds + grp];
        rb.z[tn] = (uint32_t)mem.qzeros[(size_t)ncol[tn] * mem.ldz + (grp >> 3)];
      } else {
        rb.s[tn] = __builtin_nondeterministic_value(rb.s[tn]);
        rb.z[tn] = __builtin_nondeterministic_value(rb.z[tn]);
      }
    }
  };
  auto stage_b = [&](const BRegs& rb, int i) {
    if (bulk) {
      const int start = min(first + (i & ~7), sblocks - 8);  // runs of eight from the wave's first super-block
      if (start != run_start) fetch_run(start);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous super-block are done
    __builtin_amdgcn_wave_barrier();
    const int j = first + i - run_start;
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<u32x4*>(btile + (tn * 32 + q * 8 + (lane >> 3)) * kSegStride + (lane & 7) * 16) = rb.b[tn * 4 + q];
      if constexpr (kRaw) {
        if (bulk) {
          const u32x4 rs = (j & 4) ? run_s2[tn] : run_s[tn];
          cur_s[tn] = (j & 2) ? ((j & 1) ? rs.w : rs.z) : ((j & 1) ? rs.y : rs.x);
          cur_z[tn] = (uint32_t)(run_z[tn] >> (8 * j)) & 0xFFu;
        } else {
          cur_s[tn] = rb.s[tn];
          cur_z[tn] = (rb.z[tn] >> (4 * ((2 * (first + i)) & 7))) & 0xFFu;
        }
      } else if (bulk) {
        const u32x4 rs = run_s[tn];
        const uint32_t sp = (j & 4) ? ((j & 2) ? rs.w : rs.z) : ((j & 2) ? rs.y : rs.x);
        cur_s[tn] = (j & 1) ? sp >> 16 : sp & 0xFFFFu;
        cur_z[tn] = (uint32_t)(run_z[tn] >> (8 * j)) & 0xFu;
      } else {
        cur_s[tn] = rb.s[tn];
        cur_z[tn] = nibble(rb.z[tn], (((first + i) * 256 + lh * 128) >> g.gs_shift) & 7);
      }
    }
  };
  // jj: first or second half of every lane's 128 columns: the 64-column halves jj of both groups -- kRaw: both halves of
  // group jj
  auto issue_a = [&](int i, int jj, ARegs& ra) {
    const int kbase = min(first + i, sblocks - 1) * 256 + jj * (kRaw ? 128 : 64) + (lane & 7) * 8;
    constexpr int kSegCols = kRaw ? 64 : 128;  // columns between the two segments of a token row
#pragma unroll
    for (int q = 0; q < kMT * 8; ++q) {
      const int seg = q * 8 + (lane >> 3);             // (token row, half of the super-block)
      const int row = min(seg >> 1, g.M - 1);
      // loads whose four token rows all lie past M are skipped, and so is their staging: those rows of the tile keep
      // whatever the LDS held, and the accumulator rows they feed are never stored
      if (q * 4 < g.M) ra.a[q] = *reinterpret_cast<const u32x4*>(g.x + (size_t)row * g.K + kbase + (seg & 1) * kSegCols);
      else ra.a[q] = __builtin_nondeterministic_value(ra.a[q]);  // no value carried round the loop: nothing to wait for
    }
  };
  auto stage_a = [&](const ARegs& ra) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous half are done
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < kMT * 8; ++q)  // staged in the order of the weight nibbles, so that fragment reads need no permute
      if (q * 4 < g.M) {
        if constexpr (kRaw) {
          // sixteen lanes hold the 128 columns of the group for token row 4 q + lane / 16: their sum, in fp32
          const h8 v = __builtin_bit_cast(h8, ra.a[q]);
          const h2 ones = {(half_t)1.f, (half_t)1.f};
          float sum = __builtin_amdgcn_fdot2(h2{v[0], v[1]}, ones, 0.f, false);
          sum = __builtin_amdgcn_fdot2(h2{v[2], v[3]}, ones, sum, false);
          sum = __builtin_amdgcn_fdot2(h2{v[4], v[5]}, ones, sum, false);
          sum = __builtin_amdgcn_fdot2(h2{v[6], v[7]}, ones, sum, false);
          sum = row16_total(sum);
          if ((lane & 15) == 0) asig[q * 4 + (lane >> 4)] = sum;
          // the odd nibbles come out of the mask as code * 2^-20: their activations carry the 1/16 (exact but for
          // values below 2^-10, which lose bits worth 2^-25 and less)
          u32x4 o = __builtin_bit_cast(u32x4, nibble_order(ra.a[q]));
          const h2 sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
          o.y = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.y) * sixteenth);
          o.w = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.w) * sixteenth);
          *reinterpret_cast<u32x4*>(atile + (q * 8 + (lane >> 3)) * kSegStride + (lane & 7) * 16) = o;
        } else {
          *reinterpret_cast<h8*>(atile + (q * 8 + (lane >> 3)) * kSegStride + (lane & 7) * 16) = nibble_order(ra.a[q]);
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // kRaw: group gi of the super-block, all of it: quarters lh and 2 + lh of its codes against the staged group
  auto compute_raw = [&](int gi) {
    f16v ag[kMT][kNT];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      h8 bf[kNT][4];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        const u32x4 bw = *reinterpret_cast<const u32x4*>(btile + (tn * 32 + ln) * kSegStride + gi * 64 + lh * 32 + jj * 16);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t wd = bw[t], hi = wd >> 8;
          bf[tn][t] = __builtin_bit_cast(h8, u32x4{wd & 0x000F000Fu, wd & 0x00F000F0u, hi & 0x000F000Fu, hi & 0x00F000F0u});
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int tm = 0; tm < kMT; ++tm) {
          const h8 af = *reinterpret_cast<const h8*>(atile + (((tm * 32 + ln) * 2 + lh) * kSegStride) + (4 * jj + t) * 16);
#pragma unroll
          for (int tn = 0; tn < kNT; ++tn) {
            if (jj == 0 && t == 0) {
              const f16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              ag[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf[tn][t], zero, 0, 0, 0);
            } else {
              ag[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf[tn][t], ag[tm][tn], 0, 0, 0);
            }
          }
        }
      }
    }
    // scale and zero-point of the group on its sum: rows 8 k + 4 lh + e of the tile sit in registers 4 k + e
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      const float sc = (float)__builtin_bit_cast(half_t, (uint16_t)((cur_s[tn] >> (16 * gi)) & 0xFFFFu));
      const float sf = sc * 0x1p24f, sz = -sc * (float)((cur_z[tn] >> (4 * gi)) & 0xFu);
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (tm * 32 + 8 * k < g.M) {
            const f4 sg = *reinterpret_cast<const f4*>(asig + tm * 32 + 8 * k + 4 * lh);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[tm][tn][4 * k + e] = __builtin_fmaf(sf, ag[tm][tn][4 * k + e], __builtin_fmaf(sz, sg[e], acc[tm][tn][4 * k + e]));
          }
        }
      }
    }
  };
  auto compute = [&](int i, int j) {
    h8 bf[kNT][4];
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      const half_t z = (half_t)(float)cur_z[tn];
      const half_t zl = (half_t)(-1024.0f) - z, zh = (half_t)(-64.0f) - z;
      const h2 zb_lo = {zl, zl}, zb_hi = {zh, zh};
      const h2 s2 = bitcast_u32<h2>(cur_s[tn] | (cur_s[tn] << 16));
      const u32x4 bw = *reinterpret_cast<const u32x4*>(btile + (tn * 32 + ln) * kSegStride + lh * 64 + j * 16);
      bf[tn][0] = dequant_word_sk(bw.x, zb_lo, zb_hi, s2);
      bf[tn][1] = dequant_word_sk(bw.y, zb_lo, zb_hi, s2);
      bf[tn][2] = dequant_word_sk(bw.z, zb_lo, zb_hi, s2);
      bf[tn][3] = dequant_word_sk(bw.w, zb_lo, zb_hi, s2);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm) {
        const h8 af = *reinterpret_cast<const h8*>(atile + (((tm * 32 + ln) * 2 + lh) * kSegStride) + (4 * (j & 1) + t) * 16);
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf[tn][t], acc[tm][tn], 0, 0, 0);
      }
    }
  };

  // Weights one super-block ahead, activations half a super-block ahead, both in registers in load order and moved to
  // the LDS tiles when their turn begins.  The weight loads go out behind the activation loads of the first half:
  // waiting for those activations then leaves the weights in flight.
#define GLOWQ_PIN_LOADS() asm volatile("" ::: "memory")
  BRegs B;
  ARegs A;
  if (bulk) fetch_run(min(first, sblocks - 8));
  issue_b(0, B);
  issue_a(0, 0, A);
  GLOWQ_PIN_LOADS();
  for (int i = 0; i < mine; ++i) {
    stage_b(B, i); stage_a(A);
    issue_a(i, 1, A); issue_b(i + 1, B); GLOWQ_PIN_LOADS();
    if constexpr (kRaw) compute_raw(0); else { compute(i, 0); compute(i, 1); }
    stage_a(A);
    issue_a(i + 1, 0, A); GLOWQ_PIN_LOADS();
    if constexpr (kRaw) compute_raw(1); else { compute(i, 2); compute(i, 3); }
  }
#undef GLOWQ_PIN_LOADS
  if constexpr (kProj) {
    // the correction behind the weights: acc_w + alpha (r . L^T) = alpha (acc_w / alpha + r . L^T)
    if (corrected && wave < lblocks) {
      int seen = 0;
      if (lane == 0) {
        for (unsigned spins = 0; !seen && spins <= g.spin && g.spin != 0xFFFFFFFFu; ++spins) {
          seen = (__hip_atomic_load(g.pub, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & kTagMask) == tag;
          if (!seen) __builtin_amdgcn_s_sleep(2);
        }
      }
      seen = __builtin_amdgcn_readfirstlane(seen);
      if (g.alpha != 1.0f) scale_acc(1.0f / g.alpha);
      correction(seen != 0);
      if (g.alpha != 1.0f) scale_acc(g.alpha);
    }
  }
  __syncthreads();  // the reduction buffer below overlays the staging tiles

  // ---- the waves' partial tiles meet in LDS: [wave][tm][tn][16 regs][64 lanes] floats; only registers and slots of
  // token rows below M take part ----------------------------------------------------------------------------------
  float* red = reinterpret_cast<float*>(smem);
  constexpr int kTile = kMT * kNT * 16 * 64;
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (tm * 32 + 8 * (i >> 2) < g.M) {
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) red[(size_t)wave * kTile + ((tm * kNT + tn) * 16 + i) * 64 + lane] = acc[tm][tn][i];
      }
  __syncthreads();
  const int slots = g.M * (32 * kNT);  // (token row, column of the workgroup's tile), column fastest
  for (int sidx = threadIdx.x; sidx < slots; sidx += blockDim.x) {
    const int m = sidx / (32 * kNT), col = sidx - m * (32 * kNT);
    const int tm = m >> 5, mm = m & 31, tn = col >> 5;
    const int reg = ((mm >> 3) << 2) | (mm & 3);
    const int at = ((tm * kNT + tn) * 16 + reg) * 64 + ((mm >> 2) & 1) * 32 + (col & 31);
    float v = 0.f;
    for (int w = 0; w < waves; ++w) v += red[(size_t)w * kTile + at];
    const int n = n0 + col;
    if (g.slices > 1) {
      g.partials[(((size_t)blockIdx.y * tiles + wg) * g.M + m) * (32 * kNT) + col] = v;
    } else if (n < mem.N) {
      const float b = mem.bias ? (float)mem.bias[n] : 0.f;
      mem.y[(size_t)m * mem.ldy + n] = (half_t)(v + b);
    }
  }
}

// Adds the K slices of skinny_group_kernel in slice order, then bias, and writes y.  One workgroup per tile.
template <int kNT>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(const SkinnyArgs g) {
  SkinnyMember mem = g.mem[0];
  int blk_base = 0;
#define GLOWQ_PICK(i)                                          \
  if (g.n_members > i && (int)blockIdx.x >= g.blk_end[i - 1]) { \
    mem = g.mem[i];                                            \
    blk_base = g.blk_end[i - 1];                               \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int n0 = ((int)blockIdx.x - blk_base) * (32 * kNT);
  const int slots = g.M * (32 * kNT);
  for (int sidx = threadIdx.x; sidx < slots; sidx += blockDim.x) {
    const int m = sidx / (32 * kNT), col = sidx - m * (32 * kNT);
    const int n = n0 + col;
    if (n >= mem.N) continue;
    float v = 0.f;
    for (int sl = 0; sl < g.slices; ++sl) v += g.partials[(((size_t)sl * gridDim.x + blockIdx.x) * g.M + m) * (32 * kNT) + col];
    const float b = mem.bias ? (float)mem.bias[n] : 0.f;
    mem.y[(size_t)m * mem.ldy + n] = (half_t)(v + b);
  }
}

// ---- host side ------------------------------------------------------------------------------------------
// The second form needs whole 256-column super-blocks and one quantisation group per 128-column half.
bool skinny_group_form(const GroupDev& g) {
  static const int env_form = getenv("GLOWQ_SKINNY_FORM") ? atoi(getenv("GLOWQ_SKINNY_FORM")) : -1;
  return (g.K & 255) == 0 && g.group_size >= 128 && env_form != 0;
}

// The raw-code form of the second form: groups of exactly 128 columns, scale rows that start on a 4-byte boundary.  Its
// arithmetic is that of the GEMV routes (weights never rounded to fp16), so the route table reports it as a route of its
// own.
bool skinny_raw_form(const GroupDev& g) {
  if (!skinny_group_form(g) || g.group_size != 128) return false;
  for (int i = 0; i < g.n_members; ++i)
    if ((g.mem[i].lds & 1) != 0 || (reinterpret_cast<uintptr_t>(g.mem[i].scales) & 3u) != 0) return false;
  return true;
}

bool skinny_supported(const GroupDev& g) {
  if (g.M < 1 || g.M > 64) return false;
  if ((g.K & 63) != 0 || (g.group_size & 31) != 0 || (g.group_size & (g.group_size - 1)) != 0) return false;
  // r is either given or still to be produced from R into r_out by the projection launch that goes ahead
  const half_t* r = g.r != nullptr ? g.r : (g.R != nullptr ? g.r_out : nullptr);
  if (r != nullptr && ((g.rank & 7) != 0 || g.rank < 8)) return false;
  if ((reinterpret_cast<uintptr_t>(g.x) & 15u) != 0) return false;
  if (r != nullptr && (reinterpret_cast<uintptr_t>(r) & 15u) != 0) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if ((reinterpret_cast<uintptr_t>(m.qweight) & 15u) != 0 || (m.ldw & 3) != 0) return false;
    if (m.L != nullptr && (reinterpret_cast<uintptr_t>(m.L) & 15u) != 0) return false;
  }
  return true;
}

// Scales and zero-points in runs of eight super-blocks: groups of 128 columns, rows of eight super-blocks or more, four
// or more super-blocks per wave, and scale rows that start on a 4-byte boundary.
static bool skinny_bulk_runs(const SkinnyArgs& a, int waves) {
  const int sblocks = a.K >> 8;
  const int sb_slice = (sblocks + a.slices - 1) / a.slices;
  if (a.gs_shift != 7 || sblocks < 8 || (sb_slice + waves - 1) / waves < 4) return false;
  for (int i = 0; i < a.n_members; ++i)
    if ((a.mem[i].lds & 1) != 0 || (reinterpret_cast<uintptr_t>(a.mem[i].scales) & 3u) != 0) return false;
  return true;
}

// ws_bytes: room behind a.partials (0: none).  The second form cuts K into slices through it where the column tiles
// alone leave half of the CUs or more without a workgroup and every wave still keeps three super-blocks and more
// (4096 outputs of K = 14336: 128 workgroups -> 2 x 128; 8 rows 16.6 -> about 14.5 us, 64 rows 41 -> about 28).
template <int kMT, int kNT, bool kGroupForm, bool kRaw = false, bool kProj = false>
static hipError_t launch_skinny_t(SkinnyArgs& a, int waves, int num_cus, size_t ws_bytes, hipStream_t stream) {
  static_assert(kGroupForm || !kRaw, "the raw-code form is a variant of the second form");
  static_assert(kGroupForm || !kProj, "only the second form computes r itself");
  int total = 0;
  for (int i = 0; i < a.n_members; ++i) {
    total += (a.mem[i].N + 32 * kNT - 1) / (32 * kNT);
    a.blk_end[i] = total;
  }
  a.slices = 1;
  static const int env_split = getenv("GLOWQ_SKINNY_SPLIT") ? atoi(getenv("GLOWQ_SKINNY_SPLIT")) : 1;
  if (kGroupForm && env_split != 0 && a.partials != nullptr && total * 2 <= num_cus) {
    const int sblocks = a.K >> 8;
    int s = num_cus / total;
    if (s > sblocks / (3 * waves)) s = sblocks / (3 * waves);
    if (s > 8) s = 8;
    const size_t per_slice = (size_t)total * a.M * (32 * kNT) * sizeof(float);
    if (per_slice > 0 && (size_t)s > ws_bytes / per_slice) s = (int)(ws_bytes / per_slice);
    // (a launch that computes r itself is not cut in two: the workgroups a second slice would bring are worth less than
    // the projection launch and the reduction launch together -- down_proj of an 8B layer, 128 column tiles, two slices
    // with both launches 20.6 us at 8 rows and 23.9 at 16, one slice with 64 / 127 producers in front 18.5 and 21.1)
    if (kProj && s == 2) s = 1;
    if (s >= 2) a.slices = s;
  }
  const bool bulk = kGroupForm && skinny_bulk_runs(a, waves);
  auto kern = !kGroupForm ? skinny_mfma_kernel<kMT, kNT>
              : bulk ? skinny_group_kernel<kMT, kNT, true, kRaw, kProj> : skinny_group_kernel<kMT, kNT, false, kRaw, kProj>;
  size_t lds = (size_t)waves * kMT * kNT * 16 * 64 * sizeof(float);
  const size_t staging = (size_t)waves * ((kMT * 64 + kNT * 32) * 144 + (kRaw ? kMT * 32 * sizeof(float) : 0));
  if (kGroupForm && lds < staging) lds = staging;
  static LdsLimit lds_limit[2];  // one per kernel this site launches
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit[bulk]); e != hipSuccess) return e;
  int grid_x = total;
  if constexpr (kProj) {
    static std::atomic<long> asked_for[2] = {{-1}, {-1}};
    static std::atomic<int> resident[2] = {{0}, {0}};
    const long shape = (long)lds * 4096 + waves * 64;
    int per_cu = 0;
    if (asked_for[bulk].load(std::memory_order_acquire) == shape) {
      per_cu = resident[bulk].load(std::memory_order_relaxed);
    } else {
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), waves * 64, lds) != hipSuccess) per_cu = 0;
      resident[bulk].store(per_cu, std::memory_order_relaxed);
      asked_for[bulk].store(shape, std::memory_order_release);
    }
    // The workgroups in front take the places the launch leaves free on the chip (its staging tiles allow one workgroup
    // per compute unit), and only where those are enough for one to one and a half blocks of r per producer: every workgroup
    // of the launch then starts at once, the producers are done long before the first wave asks for r, and no workgroup
    // with a column tile waits for a place (one that does adds its whole run time to the launch: q|k|v of an 8B layer at
    // eight rows with 257 workgroups for 256 places 11.25 us against 11.05 with the projection launch in front; fewer
    // producers with more blocks each: down_proj 32 us against 19).
    const long capacity = (long)per_cu * num_cus;
    long want = (capacity - (long)total * a.slices) & ~3L;  // (the front is padded to a multiple of four: handover.hpp)
    static const int env_producers = getenv("GLOWQ_SKINNY_PRODUCERS") ? atoi(getenv("GLOWQ_SKINNY_PRODUCERS")) : 0;
    if (env_producers > 0) want = env_producers;
    const int nblocks = ((a.rank + 3) / 4) * ((a.M + 3) / 4);  // blocks of r: four token rows by four rows of R
    if (want > nblocks) want = nblocks;
    if (want > kSkinnyMaxProducers) want = kSkinnyMaxProducers;
    // (a few producers with two blocks are as far as it goes: 4 x 8 blocks, two to a producer, on o_proj of a 14B layer
    // at 16 rows: 16.4 us against 14.3 with the projection launch; 4 x 4 blocks, 2.7 to a producer: 16.1)
    // (up to about one and a half blocks per producer pay -- 8B shapes: q|k|v at 12 rows, 96 blocks for 63 producers, 11.0
    // us against 11.7 with the projection launch; o_proj at 24 rows, 192 for 127, 11.2 against 12.4 -- two do not: q|k|v at
    // 16 rows, 128 for 63, 13.2 against 12.0)
    // Blocks a producer works on at a time (teams of four waves): one where there is a producer for every block; two, in
    // a workgroup of eight waves, where that brings all blocks of r under way at once; else, one at a time, up to about
    // one and a half per producer.  8B shapes, us, inside the launch / projection launch in front: q|k|v at 12 rows (96
    // blocks, 64 places) 9.4 / 11.7, o_proj at 24 rows (192, 128) 9.6 / 12.4; two rounds do not pay: q|k|v at 16 rows
    // with 126 slots for 128 blocks 12.4 / 11.8, o_proj of a 14B layer at 16 rows (256 blocks, 190 slots) 15.4 / 14.4.
    const int teams = (nblocks > want && waves >= 8 && nblocks <= 2 * want) ? 2 : 1;
    if (want < 1 || (nblocks > want * teams && 13 * want < 8 * nblocks && a.spin != 0xFFFFFFFFu)) return hipErrorNotReady;
    a.teams = teams;
    a.producers = (int)want;
    grid_x = front_grid(total, a.producers);
  }
  hipLaunchKernelGGL(kern, dim3(grid_x, a.slices), dim3(waves * 64), lds, stream, a);
  if constexpr (kProj) note_launch(grid_x, a.slices, waves * 64, "skinny_group_kernel<%d,%d,%d,%d,1>", kMT, kNT, (int)bulk, (int)kRaw);
  if (hipError_t e = hipGetLastError(); e != hipSuccess || a.slices == 1) return e;
  hipLaunchKernelGGL(skinny_reduce_kernel<kNT>, dim3(total), dim3(256), 0, stream, a);
  return hipGetLastError();
}

// The most workspace the split of K above asks for: it cuts only while slices x column tiles stay within num_cus
// workgroups, and a split launch has 32-column tiles (the 64-column ones belong to groups that fill the chip without it):
// one 32-column fp32 tile per token row for each of num_cus workgroups.
size_t skinny_split_workspace_bytes(int M, int num_cus) { return M > 4 ? (size_t)num_cus * (size_t)M * 32 * sizeof(float) : 0; }

hipError_t launch_skinny(GroupDev& g, int num_cus, hipStream_t stream, bool raw) {
  SkinnyArgs a;
  a.x = g.x;
  a.r = g.r;
  a.n_members = g.n_members;
  a.M = g.M;
  a.K = g.K;
  a.rank = g.rank;
  a.gs_shift = __builtin_ctz(g.group_size);
  a.alpha = g.alpha;
  a.slices = 1;
  const bool ws_ok = g.ws != nullptr && (reinterpret_cast<uintptr_t>(g.ws) & 15u) == 0;
  a.partials = ws_ok ? static_cast<float*>(g.ws) : nullptr;
  size_t ws_bytes = ws_ok ? g.ws_bytes : 0;
  // the launch computes r itself (run_group set g.pub to the head of the workspace): the partial tiles lie behind the
  // hand-over words
  const bool proj = g.pub != nullptr;
  a.R = g.R;
  a.r_out = g.r_out;
  a.pub = g.pub;
  a.spin = g.pub_mute ? 0xFFFFFFFFu : g.pub_spin;
  a.producers = 0;
  a.teams = 1;
  if (proj) {
    if (!ws_ok || ws_bytes < kSkinnyHandoverBytes) return hipErrorNotReady;
    a.r = nullptr;
    a.partials = reinterpret_cast<float*>(static_cast<unsigned char*>(g.ws) + kSkinnyHandoverBytes);
    ws_bytes -= kSkinnyHandoverBytes;
  }
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    SkinnyMember& s = a.mem[i];
    s.qweight = m.qweight;
    s.scales = m.scales;
    s.qzeros = m.qzeros;
    s.L = m.L;
    s.bias = m.bias;
    s.y = m.y;
    s.N = m.N;
    s.ldw = m.ldw;
    s.lds = m.lds;
    s.ldz = m.ldz;
    s.ldy = m.ldy;
  }
  static const int env_waves = getenv("GLOWQ_SKINNY_WAVES") ? atoi(getenv("GLOWQ_SKINNY_WAVES")) : 0;
  int waves = (env_waves >= 1 && env_waves <= 8) ? env_waves : 8;
  if (skinny_group_form(g)) {
    // two column tiles per wave halve the activation traffic, one gives twice the workgroups: the wide tile only
    // where there are columns to fill the chip with it
    long cols = 0;
    for (int i = 0; i < g.n_members; ++i) cols += g.mem[i].N;
    const bool wide = cols >= 64L * num_cus;
    if (env_waves < 1) waves = wide ? 4 : (g.M <= 32 ? 8 : 6);  // staging tiles: 18 / 13.5 / 22.5 KB of LDS per wave
    if (waves > (g.K >> 8)) waves = g.K >> 8;
    if (raw && !skinny_raw_form(g)) return hipErrorInvalidValue;
    if (proj) {
      // (the narrow tile at up to 32 rows, four waves and more: the shapes whose launch leaves room on the chip)
      if (g.M > 32 || wide || waves < 4) return hipErrorNotReady;
      return raw ? launch_skinny_t<1, 1, true, true, true>(a, waves, num_cus, ws_bytes, stream)
                 : launch_skinny_t<1, 1, true, false, true>(a, waves, num_cus, ws_bytes, stream);
    }
    if (g.M <= 32) {
      if (raw) return wide ? launch_skinny_t<1, 2, true, true>(a, waves, num_cus, ws_bytes, stream) : launch_skinny_t<1, 1, true, true>(a, waves, num_cus, ws_bytes, stream);
      return wide ? launch_skinny_t<1, 2, true>(a, waves, num_cus, ws_bytes, stream) : launch_skinny_t<1, 1, true>(a, waves, num_cus, ws_bytes, stream);
    }
    if (!wide) {
      if (waves > 6) waves = 6;
      // 2 x 2 tiles do not fit the register file with the staging
      return raw ? launch_skinny_t<2, 1, true, true>(a, waves, num_cus, ws_bytes, stream) : launch_skinny_t<2, 1, true>(a, waves, num_cus, ws_bytes, stream);
    }
    // many columns and more than 32 rows: two passes of 32 rows over the wide tile beat one pass over the narrow one
    for (int m0 = 0; m0 < g.M; m0 += 32) {
      SkinnyArgs c = a;
      c.M = g.M - m0 < 32 ? g.M - m0 : 32;
      c.x = a.x + (size_t)m0 * g.K;
      c.r = a.r ? a.r + (size_t)m0 * g.rank : nullptr;
      for (int i = 0; i < g.n_members; ++i) c.mem[i].y = a.mem[i].y + (size_t)m0 * a.mem[i].ldy;
      hipError_t e = raw ? launch_skinny_t<1, 2, true, true>(c, waves, num_cus, ws_bytes, stream) : launch_skinny_t<1, 2, true>(c, waves, num_cus, ws_bytes, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  if (raw) return hipErrorInvalidValue;
  if (proj) return hipErrorNotReady;
  const int kblocks = g.K >> 6;
  if (waves > kblocks) waves = kblocks;
  if (g.M <= 32) return launch_skinny_t<1, 2, false>(a, waves, num_cus, ws_bytes, stream);
  return launch_skinny_t<2, 2, false>(a, waves, num_cus, ws_bytes, stream);
}

}  // namespace glowq
