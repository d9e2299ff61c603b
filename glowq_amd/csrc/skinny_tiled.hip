// Matrix-core kernel for a handful of token rows (5..64, from 2 on the longest streams) on members that bring the tiled copy of their weights
// (tiled.hpp): the weights are streamed once, every 16-byte load of a wave is one contiguous kilobyte and lands in
// the lanes' registers as the B operand of v_mfma_f32_32x32x16_f16 -- no pass through LDS, no per-lane scale and
// zero-point gather (both ride in the stream).
//
// Arithmetic: that of the reference's GEMV (src/cuda_w4a16/csrc/gemv_w4a16.cu:96-112, which the reference uses up to 128
// token rows): the weight (code - zero) * scale is never rounded to fp16.  The codes go to the matrix cores as they are
// -- a nibble masked in place is the fp16 subnormal code * 2^-24 (or code * 2^-20; the activations of those columns
// are staged divided by 16) -- the eight instructions of a 128-column half leave sum code * x per (token row, output
// row), a ninth adds -zero * sum x (the per-row sums of the activations come as one more A fragment), and the scale
// is applied to that sum in fp32: y += scale * 2^24 * sum.  Five vector instructions per code word instead of the
// thirteen a dequantisation to fp16 takes: the vector ALUs, not memory, bound the dequantising form.
// (The division by 16 is exact for |x| >= 2^-10; below, x / 16 is a subnormal and x is rounded to a multiple of 2^-20,
// an absolute error of 2^-21 and less.  The row sums are carried as two halves, good to 2^-22 of their value.)
//
// A workgroup owns 32 cw output columns of one member (a row block of 32 per consumer wave) and all token rows.  Its
// waves come in K groups that walk contiguous parts of the K range in step and meet in LDS at the end; a K group is
// `cw` consumer waves (four as a rule; more where that brings the column tiles down to one per compute unit) and kPW
// producer waves.
//   * Consumers keep kD sets of weight registers in rotation: the set of super-block v is refilled with super-block
//     v + kD as soon as its words have been masked, so up to kD - 1 super-blocks of a wave are in flight while it
//     computes.  They wait for nothing but their weights.
//   * Producers load the activations of the next super-block (token rows x 512 bytes) in memory order (the tiled copy
//     holds the nibbles of a word in the order the masks deliver them: no permutation), divide the pairs at positions
//     2, 3 and 6, 7 of every octet by 16, sum every row's two
//     128-column halves in fp32, and leave all of it in the LDS stage the consumers do not read (528-byte rows:
//     conflict-free 16-byte reads).  One barrier per super-block.  A wave's loads return in order: a consumer that
//     fetched activations as well would have to drain its weight requests with every step.
// The correction is a K-extension behind the weights: in the last rotation the sets are refilled with the blocks of
// the tiled left factor (fp16, already in B-operand order), r follows the last super-block through the stages, and
// acc += alpha * (r . L^T) from an accumulator of its own.
// kProj: the launch computes r = x R^T itself.  Workgroups in front of the grid (roles dealt as in handover.hpp) produce
// blocks of four token rows by four rows of R in the arithmetic of shared_proj_block_kernel and write them to r_out with
// stores that pass the caches private to a part of the chip (two blocks at a time where the workgroup has eight waves
// and more), each raises its flag when its stores are acknowledged, and the first of them turns the flags into one ready
// word.  The producer waves of the other workgroups look for that word when
// they are about to send r through the stages -- during the last super-block, so the producers in front have the whole
// weight stream to get there -- and read r with loads that pass those caches; one that does not see the word within its
// bound computes the pieces of r it would have loaded, so every wave ends whatever becomes of the workgroups in front.
// Few column tiles (o_proj, down_proj): K is also cut into gridDim.y slices, each workgroup leaves its fp32 tile in the
// caller's workspace and skinny_tiled_reduce_kernel adds the slices in order.  More than 32 token rows: two row tiles
// per wave, every code word feeds two matrix instructions.
#include <atomic>
#include <cstdlib>

#include <type_traits>

#include "common.hpp"
#include "handover.hpp"
#include "proj_block.hpp"
#include "tiled.hpp"

namespace glowq {

struct TileMember {
  const unsigned char* wt;  // tiled weights (tiled.hpp)
  const unsigned char* lt;  // tiled left factor or nullptr
  const half_t* bias;
  half_t* y;
  int N, ldy;
  int col0;                 // first column of the member in a row of the partial buffer (members padded to 128)
};

struct TileArgs {
  const half_t* r;  // [M, rank] or nullptr
  TileMember mem[GLOWQ_MAX_MEMBERS];
  int blk_end[GLOWQ_MAX_MEMBERS];
  int n_members;
  int M, K, rank;
  float alpha;
  int slices;       // gridDim.y
  float* partials;  // [slice][M][ldp] fp32 when slices > 1
  int ldp;
  int tiles;        // column tiles of the whole group: the grid's x extent
  int cw;           // consumer waves per K group: a tile is 32 cw columns
  // kProj (the launch computes r itself; `r` then points at r_out)
  const half_t* R;          // [rank, K]
  half_t* r_out;            // [M, rank]
  unsigned long long* pub;  // [0]: the ready word; [kTiledFlags + p]: the flag of producer p
  unsigned spin;            // polls of the ready word before a producer wave computes its pieces of r itself
  int producers;            // workgroups in front that produce r
  int teams;                // blocks of r a producer works on at a time: teams of four waves (1 or 2)
};
constexpr int kTiledFlags = 512;  // the producers' flags lie 4096 bytes behind the ready word
constexpr int kTiledMaxProducers = 512;
constexpr size_t kTiledHandoverBytes = (size_t)(kTiledFlags + kTiledMaxProducers) * 8;
// blocks of r a producer in front may have to compute (gate|up of a 14B layer, rank 256, 35 producers: 3.7 blocks each at
// eight rows 26.8 us against 30.9 with the projection launch, 5.5 at twelve 27.4 against 31.3, 7.3 at sixteen 30.5 to 31.5
// against 31.5)
constexpr int kTiledProjBlocks = 6;

namespace {

// The code of column k of a word (nibble k in the canonical buffers) moves to nibble (0,4,1,5,2,6,3,7)[k]: the four
// masks of the kernels then deliver the eight codes in column order.
__device__ __forceinline__ uint32_t mask_order_word(uint32_t w) {
  uint32_t o = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) o |= ((w >> (4 * k)) & 0xFu) << (4 * ((k >> 1) + 4 * (k & 1)));
  return o;
}

// total over a row of 16 lanes, in every lane of it
__device__ __forceinline__ float row16_total_t(float v) {
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

constexpr int kRowBytes = 528;  // 512 bytes of a token row's super-block + 16: rows 8 apart share no bank
constexpr int kD = 4;           // weight register sets in rotation
#ifndef GLOWQ_TILED_AUX
#define GLOWQ_TILED_AUX 2
#endif
constexpr int kStreamAux = GLOWQ_TILED_AUX;  // cache policy of the weight loads: non-temporal, every byte is used once

}  // namespace

#ifndef GLOWQ_TDBG
#define GLOWQ_TDBG 0
#endif
#if GLOWQ_TDBG & 32
__device__ unsigned long long g_tstamps[65536 * 32];
#define GLOWQ_STAMP(i) do { if (lane == 0 && !producer) g_tstamps[(((size_t)blockIdx.x * gridDim.y + blockIdx.y) * 16 + (threadIdx.x >> 6)) * 32 + (i)] = wall_clock64(); } while (0)
#else
#define GLOWQ_STAMP(i) do { } while (0)
#endif

// kRows: token rows a K group stages (8, 16, 32 or 64).  kWk: K groups per workgroup.  kPW: producer waves per K group.
// The leading scalar arguments arrive in registers with the wave (kernel-argument preload): what a workgroup of the
// first member needs to request its first weights and activations, without a round trip to the argument buffer.
// Consumer waves a K group may have and the workgroup size that goes with it: 768 threads at most, 512 where a wave
// holds two row tiles (their registers do not fit three waves on a SIMD).
constexpr int tiled_max_cw(int rows, int wk, int pw) { return wk > 1 ? 4 : (rows > 32 ? 8 - pw : 12 - pw); }
constexpr int tiled_max_threads(int rows, int wk, int pw) { return (tiled_max_cw(rows, wk, pw) + pw) * 64 * wk; }

template <int kRows, int kWk, int kPW, bool kProj = false>
__global__ __launch_bounds__(tiled_max_threads(kRows, kWk, kPW))
void skinny_tiled_kernel(const half_t* __restrict__ x, const int M, const int K, const int slices,
                         const unsigned char* __restrict__ wt0, const int blk_end0, const int N0, const int cw, const TileArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_all[];
  constexpr int kMT = kRows > 32 ? 2 : 1;        // 32-row tiles per consumer wave
  constexpr int kPQ = (kRows + 2 * kPW - 1) / (2 * kPW);  // 16-byte pieces of a super-block of x per producer thread
  constexpr bool kRagged = kPQ * 2 * kPW != kRows;       // three producer waves: the last pass covers part of the rows
  constexpr int kSigBytes = kRows * 16;          // per 128-column half: a 16-byte fragment of sums per token row
  constexpr int kStage = kRows * kRowBytes + 2 * kSigBytes;
  constexpr int kLiveRegs = kRows >= 32 ? 16 : (kRows >= 16 ? 8 : 4);  // accumulator registers of rows that exist
  const int group_threads = (cw + kPW) * 64;  // the consumer waves, then the producer waves
  const int gk = kWk > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >= group_threads ? 1 : 0) : 0;
  static_assert(kWk <= 2, "gk is a comparison");
  const int tig = (int)threadIdx.x - gk * group_threads;  // thread within the K group
  const int lane = tig & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tig >> 6);
  const bool producer = wave >= cw;
  const int ln = lane & 31, lh = lane >> 5;
  unsigned char* smem = smem_all + gk * 2 * kStage;
  GLOWQ_STAMP(0);

  int tile = (int)blockIdx.x;
  unsigned long long tag = 0;
  if constexpr (kProj) {
    tag = launch_tag();
    const int front = g.producers;
    const int role = front_role(tile, front);
    if (role >= 0) {
      if (role >= front || blockIdx.y != 0) return;
      {
        // teams of four waves, each with a block of its own at a time
        const int teams = g.teams;
        if ((int)threadIdx.x >= 256 * teams) return;  // (the body's barriers count the waves that arrive)
        const int team = (int)threadIdx.x >> 8, ttid = (int)threadIdx.x & 255;
        float* part = reinterpret_cast<float*>(smem_all) + team * (4 * 16 + 16);
        const int jblocks = (g.rank + 3) >> 2;
        float* vals = part + 4 * 16;
        const int nblocks = jblocks * ((M + 3) >> 2);
        // blocks of four token rows by four rows of R, dealt round robin to the producers.  (Blocks of eight token rows,
        // half as many: 21.5 against 20.1 us at 12 rows on gate|up of an 8B layer, 32.0 against 27.5 on a 14B layer's;
        // three 16-byte pieces of every row in flight per thread instead of two, a row of 5120 columns in one round trip:
        // no difference.)
        for (int b0 = role * teams; b0 < nblocks; b0 += g.producers * teams) {
          const int b = b0 + team;
          const bool active = b < nblocks;
          const int bj = b % jblocks, bm = b / jblocks;
          proj_block_body<4, 4>(x, g.R, M, K, g.rank, 4 * bj, 4 * bm, part,
                                [&](int m, int j, float v) { vals[(m - 4 * bm) * 4 + (j - 4 * bj)] = v; }, ttid, active);
          __syncthreads();
          // pairs of neighbouring entries of a token row go out as one 32-bit store (ranks are multiples of 8)
          if (active && ttid < 8) {
            const int mi = ttid >> 1, pp = ttid & 1;
            const int m = 4 * bm + mi, j = 4 * bj + 2 * pp;
            if (m < M && j < g.rank) {
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
          __hip_atomic_store(g.pub + kTiledFlags + role, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      // the first producer is also the collector: one wave, lane l takes flags l, l + 64, ...
      if (role != 0 || threadIdx.x >= 64) return;
      bool all = false;
      for (unsigned spins = 0; !all && spins <= g.spin && g.spin != 0xFFFFFFFFu; ++spins) {
        bool mine = true;
        for (int p = (int)threadIdx.x; p < g.producers; p += 64)
          mine = mine && (__hip_atomic_load(g.pub + kTiledFlags + p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & kTagMask) == tag;
        all = __builtin_amdgcn_ballot_w64(!mine) == 0;
        if (!all) __builtin_amdgcn_s_sleep(2);
      }
      if (all && threadIdx.x == 0) __hip_atomic_store(g.pub, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (tile >= g.tiles) return;  // (a front larger than the grid behind it leaves places between its workgroups empty)
  }
  const int SB = K >> 8;
  // The workgroup's super-blocks (slice blockIdx.y of K) are dealt to its K groups in contiguous parts of `pg`; every
  // group runs the same number of steps, a whole number of rotations of the register sets.  Steps past the end of a
  // group's part read past the end of its descriptor, which returns zeros (zero codes at scale zero), and in the last
  // rotation they are skipped.
  const int per = (SB + slices - 1) / slices;
  const int s0 = min((int)blockIdx.y * per, SB), s1 = min(s0 + per, SB);
  const int pg = (s1 - s0 + kWk - 1) / kWk;
  const int sb0 = min(s0 + gk * pg, s1), sb1 = min(sb0 + pg, s1);
  const int rounds = max(1, (pg + kD - 1) / kD);
  const int steps = rounds * kD;
  const bool wg_corr = g.r != nullptr && blockIdx.y == 0;  // the first slice of a group that has an r: uniform
  const int LBall = (g.rank + 63) >> 6;                     // correction blocks of 64 rank columns

  const auto rsrc = [](const void* p, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
  };

  if (producer) {
    // ---- producer waves: the activations of step v + 1 go from registers to the stage the consumers do not read,
    // the loads of step v + 2 go out, barrier.  After the last super-block the first 256 columns of r follow through
    // the stages, then the later passes of a rank above 256.
    const int pt = tig - cw * 64;              // 0 .. 64 kPW - 1
    const int prow = pt >> 5, pcol = pt & 31;  // piece q of this thread: token row 2 kPW q + prow, 16-byte piece pcol
    const __amdgpu_buffer_rsrc_t rs_x = rsrc(x, (size_t)M * K * 2);
    const __amdgpu_buffer_rsrc_t rs_r = rsrc(g.r != nullptr ? (const void*)g.r : (const void*)x, g.r != nullptr ? (size_t)M * g.rank * 2 : 0);
    u32x4 av[kPQ];
    auto load_a = [&](bool is_r, int idx) __attribute__((always_inline)) {
      const __amdgpu_buffer_rsrc_t rs = is_r ? rs_r : rs_x;
      const uint32_t ld = (uint32_t)(is_r ? g.rank : K);
#pragma unroll
      for (int q = 0; q < kPQ; ++q) {
        const uint32_t row = (uint32_t)min(2 * kPW * q + prow, M - 1);
        av[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)((row * ld + (uint32_t)pcol * 8u) * 2u), idx * 512, 0);
      }
    };
    auto store_a = [&](int stage) __attribute__((always_inline)) {
      unsigned char* dst = smem + stage * kStage + prow * kRowBytes + pcol * 16;
      unsigned char* sig = smem + stage * kStage + kRows * kRowBytes + (pcol >> 4) * kSigBytes + prow * 16;
      const h2 ones = {(half_t)1.f, (half_t)1.f};
      const h2 sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
      for (int q = 0; q < kPQ; ++q) {
        if (kRagged && 2 * kPW * q + prow >= kRows) break;  // (whole groups of sixteen lanes: the row reduction stays among live lanes)
        // the sixteen lanes pcol / 16 hold the 128 columns of one half of the token row: their sum, in fp32
        const h8 v = __builtin_bit_cast(h8, av[q]);
        float sum = __builtin_amdgcn_fdot2(h2{v[0], v[1]}, ones, 0.f, false);
        sum = __builtin_amdgcn_fdot2(h2{v[2], v[3]}, ones, sum, false);
        sum = __builtin_amdgcn_fdot2(h2{v[4], v[5]}, ones, sum, false);
        sum = __builtin_amdgcn_fdot2(h2{v[6], v[7]}, ones, sum, false);
        sum = row16_total_t(sum);
        u32x4 o = av[q];
        o.y = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.y) * sixteenth);
        o.w = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.w) * sixteenth);
        *reinterpret_cast<u32x4*>(dst + 2 * kPW * q * kRowBytes) = o;
        if ((pcol & 15) == 0) {
          // sum * 2^-8 as two halves (the zero-point fragment carries -zero * 2^-16)
          const float sc = sum * 0.00390625f;
          const half_t hi = (half_t)sc;
          const half_t lo = (half_t)(sc - (float)hi);
          const uint32_t pr = (uint32_t)__builtin_bit_cast(uint16_t, hi) | ((uint32_t)__builtin_bit_cast(uint16_t, lo) << 16);
          *reinterpret_cast<u32x4*>(sig + 2 * kPW * q * 16) = u32x4{pr, pr, pr, pr};
        }
      }
    };
    // kProj: the first 256 columns of r from r_out once the ready word is up (loads that pass the caches the producers'
    // stores passed); without the word within the bound, the thread computes the eight entries of each of its pieces
    // `polls`: how often the wave looks before it gives up (one look where it may come back later).  True: the loads
    // are out.
    auto ask_r_handed = [&](unsigned polls) __attribute__((always_inline)) -> bool {
      int seen = 0;
      if (lane == 0) {
        for (unsigned spins = 0; !seen && spins < polls && g.spin != 0xFFFFFFFFu; ++spins) {
          seen = (__hip_atomic_load(g.pub, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & kTagMask) == tag;
          if (!seen && spins + 1 < polls) __builtin_amdgcn_s_sleep(2);
        }
      }
      seen = __builtin_amdgcn_readfirstlane(seen);
      if (seen) {
#pragma unroll
        for (int q = 0; q < kPQ; ++q) {
          const uint32_t row = (uint32_t)min(2 * kPW * q + prow, M - 1);
          av[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_r, (int)((row * (uint32_t)g.rank + (uint32_t)pcol * 8u) * 2u), 0, 16);
        }
      }
      return seen != 0;
    };
    auto load_r_handed = [&]() __attribute__((always_inline)) {
      if (ask_r_handed(g.spin == 0xFFFFFFFFu ? 0u : g.spin + 1u)) return;
      for (int q = 0; q < kPQ; ++q) {
        const int row = min(2 * kPW * q + prow, M - 1);
        h8 own;
        for (int e = 0; e < 8; ++e) {
          const int j = pcol * 8 + e;
          float a = 0.f;
          if (j < g.rank) {
            const half_t* Rrow = g.R + (size_t)j * K;
            const half_t* xrow = x + (size_t)row * K;
            for (int kk = 0; kk < K; ++kk) a = __builtin_fmaf((float)Rrow[kk], (float)xrow[kk], a);
          }
          own[e] = (half_t)a;
        }
        av[q] = __builtin_bit_cast(u32x4, own);
      }
    };
    load_a(false, min(sb0, SB - 1));
    store_a(0);
    load_a(false, min(sb0 + 1, SB - 1));
    __syncthreads();
    bool have_r = false;
    for (int i = 0; i < steps; ++i) {
#if !(GLOWQ_TDBG & 8)
      if constexpr (kProj) {
        // r that was not there a step earlier is waited for during the last super-block, for the stage that super-block
        // does not read
        if (i + 1 == steps && wg_corr && gk == 0 && !have_r) load_r_handed();
      }
      store_a((i + 1) & 1);                                   // step i + 1's activations (or r after the last step)
      const bool next_r = i + 2 >= steps;
      if constexpr (kProj) {
        if (!next_r) load_a(false, min(sb0 + i + 2, SB - 1));
        // where the other form asks for r, one look: as a rule the workgroups in front are long done
        else if (i + 2 == steps && wg_corr && gk == 0) have_r = ask_r_handed(1u);
      } else {
        load_a(next_r, next_r ? 0 : min(sb0 + i + 2, SB - 1));  // (past the last step: r once more, never stored)
      }
#endif
      __syncthreads();
    }
    if (wg_corr) {
      for (int pass = 1; pass * kD < LBall; ++pass) {
        __syncthreads();
        load_a(true, pass);
        store_a(0);
        __syncthreads();
      }
    }
    if constexpr (kWk > 1) {
      __syncthreads();
      __syncthreads();
    }
    return;
  }

  // ---- consumer waves -----------------------------------------------------------------------------------------------
  // the member: the first one from the leading arguments, the others from the argument buffer
  const unsigned char* wt = wt0;
  int mem_N = N0, blk_base = 0, mi = 0;
  if (tile >= blk_end0) {
#pragma unroll
    for (int i = 1; i < GLOWQ_MAX_MEMBERS; ++i)
      if (i < g.n_members && tile >= g.blk_end[i - 1]) {
        wt = g.mem[i].wt;
        mem_N = g.mem[i].N;
        blk_base = g.blk_end[i - 1];
        mi = i;
      }
  }
  const int rb = (tile - blk_base) * cw + wave;  // this wave's row block of the member
  const bool live = rb < ((mem_N + 31) >> 5);   // a wave past the member's rows still meets the barriers
  // chunk (rb, sb) lies at (sb * RB + rb) * kChunk: the descriptor starts at the wave's chunk of super-block 0 and ends
  // behind its chunk of the group's last super-block
  const int chunk_stride = ((mem_N + 31) >> 5) * tiled::kChunk;
  const __amdgpu_buffer_rsrc_t rs_w = rsrc(wt + (size_t)(live ? rb : 0) * tiled::kChunk, live && sb1 > 0 ? (size_t)(sb1 - 1) * chunk_stride + tiled::kChunk : 0);
  const int b_off = lane * 16;

  struct BSet {
    u32x4 w[4];
    u32x2 side;  // the lane's column: (scale | -zero * 2^-16) of the two halves
  };
  BSet bs[kD];
  auto request = [&](BSet& b, int sbq) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j) b.w[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, b_off + j * 1024, sbq * chunk_stride, kStreamAux);
    b.side = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_w, ln * 8, sbq * chunk_stride + tiled::kCodeBytes, kStreamAux));
  };
  // two super-blocks up front, the other two once the first activations are staged: with all four at once the whole
  // chip asks for half a long matrix before any wave can begin
  request(bs[0], sb0);
  request(bs[1], sb0 + 1);
  GLOWQ_STAMP(1);

  // a member without a left factor (GlowQ-S) reads zeros for its correction blocks
  const TileMember mem = g.mem[mi];
  const bool has_l = wg_corr && gk == 0 && mem.lt != nullptr && live;
  const __amdgpu_buffer_rsrc_t rs_l = rsrc(has_l ? mem.lt + (size_t)rb * LBall * tiled::kLChunk : wt, has_l ? (size_t)LBall * tiled::kLChunk : 0);

  f16v acc[kMT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[tm][i] = 0.f;
  const uint32_t half0 = lh == 0 ? 0xFFFFFFFFu : 0u;  // the zero-point fragment lives in the first lane half
  const int arow = kRows >= 32 ? ln : (ln & (kRows - 1));
  const int arow_off = arow * kRowBytes + 128 * lh;
  const int sig_off = kRows * kRowBytes + arow * 16;

  // One super-block: the codes of the register set `b` against the staged rows, half by half.
  // kRefill: each register of the set is refilled with super-block sb_next as soon as its words have been masked.
  auto compute = [&](int sb_next, int stage, BSet& b, auto refill_const) __attribute__((always_inline)) {
    constexpr bool kRefill = decltype(refill_const)::value;
    const unsigned char* st = smem + stage * kStage;
    const u32x2 side = b.side;
#if GLOWQ_TDBG & 1
    {
      uint32_t f = side.x ^ side.y;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u32x4 raw = b.w[j];
        if constexpr (kRefill) b.w[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, b_off + j * 1024, sb_next * chunk_stride, kStreamAux);
        f ^= raw.x ^ raw.y ^ raw.z ^ raw.w;
      }
      acc[0][0] += __builtin_bit_cast(float, f & 0x3FFFFFFFu) + *reinterpret_cast<const float*>(st + arow_off);
      if constexpr (kRefill)
        b.side = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_w, ln * 8, sb_next * chunk_stride + tiled::kCodeBytes, kStreamAux));
      return;
    }
#endif
#pragma unroll
    for (int gh = 0; gh < 2; ++gh) {
      f16v pg[kMT];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const u32x4 raw = b.w[2 * gh + p];
        if constexpr (kRefill) b.w[2 * gh + p] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, b_off + (2 * gh + p) * 1024, sb_next * chunk_stride, kStreamAux);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t wd = raw[i], hi = wd >> 8;
          const h8 bf = __builtin_bit_cast(h8, u32x4{wd & 0x000F000Fu, wd & 0x00F000F0u, hi & 0x000F000Fu, hi & 0x00F000F0u});
#pragma unroll
          for (int tm = 0; tm < kMT; ++tm) {
            const h8 af = *reinterpret_cast<const h8*>(st + arow_off + tm * 32 * kRowBytes + 256 * gh + 64 * p + 16 * i);
            if (p == 0 && i == 0) {
              const f16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              pg[tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, zero, 0, 0, 0);
            } else {
              pg[tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, pg[tm], 0, 0, 0);
            }
          }
        }
      }
      // the zero-point: k values 0 and 1 of the first lane half carry -zero * 2^-16 against the row's sum * 2^-8 (hi, lo)
      const uint32_t sw = side[gh];
      const h8 bz = __builtin_bit_cast(h8, u32x4{__builtin_amdgcn_perm(sw, sw, 0x03020302u) & half0, 0u, 0u, 0u});
      const float sf = (float)__builtin_bit_cast(half_t, (uint16_t)(sw & 0xFFFFu)) * 0x1p24f;
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm) {
        const h8 az = *reinterpret_cast<const h8*>(st + sig_off + tm * 32 * 16 + gh * kSigBytes);
        pg[tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(az, bz, pg[tm], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < kLiveRegs; ++i) acc[tm][i] = __builtin_fmaf(sf, pg[tm][i], acc[tm][i]);
      }
    }
    if constexpr (kRefill)
      b.side = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_w, ln * 8, sb_next * chunk_stride + tiled::kCodeBytes, kStreamAux));
  };

  __syncthreads();
  request(bs[2], sb0 + 2);
  request(bs[3], sb0 + 3);
  GLOWQ_STAMP(2);

  // step d of a rotation at super-block sb: compute on stage d % 2; barrier.  Last rotation: a step past the group's
  // part is skipped, and the sets are refilled with the blocks of the tiled left factor (set q: block q; past the rank
  // they lie past the end of the descriptor).
  auto step = [&](int sb, auto d_const, auto last_const) __attribute__((always_inline)) {
    constexpr int d = decltype(d_const)::value;
    constexpr bool kLast = decltype(last_const)::value;
    if constexpr (kLast) {
      if (sb < sb1) compute(0, d & 1, bs[d], std::false_type{});
#pragma unroll
      for (int t = 0; t < 4; ++t) bs[d].w[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_l, b_off + t * 1024, d * tiled::kLChunk, 0);
    } else {
      compute(sb + kD, d & 1, bs[d], std::true_type{});
    }
    GLOWQ_STAMP(8 + min(sb - sb0, 11) * 2);
    __syncthreads();
    GLOWQ_STAMP(9 + min(sb - sb0, 11) * 2);
  };
  using std::integral_constant;
  int sb = sb0;
  for (int rd = 0; rd < rounds - 1; ++rd, sb += kD) {
    step(sb, integral_constant<int, 0>{}, std::false_type{});
    step(sb + 1, integral_constant<int, 1>{}, std::false_type{});
    step(sb + 2, integral_constant<int, 2>{}, std::false_type{});
    step(sb + 3, integral_constant<int, 3>{}, std::false_type{});
  }
  GLOWQ_STAMP(3);
  step(sb, integral_constant<int, 0>{}, std::true_type{});
  GLOWQ_STAMP(4);
  step(sb + 1, integral_constant<int, 1>{}, std::true_type{});
  step(sb + 2, integral_constant<int, 2>{}, std::true_type{});
  step(sb + 3, integral_constant<int, 3>{}, std::true_type{});

  // ---- the correction: set q holds block q of the tiled left factor (B fragments of its four k-steps as they are),
  // stage 0 the first 256 columns of r.  Ranks above 256 take further passes, each with its loads in the open.  K groups
  // other than the first hold zeros in their sets.
  if (wg_corr) {
    f16v acc2[kMT];
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc2[tm][i] = 0.f;
    for (int pass = 0; pass * kD < LBall; ++pass) {
      if (pass > 0) {
        __syncthreads();  // the fragment reads of the pass before are done
#pragma unroll
        for (int q = 0; q < kD; ++q)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            bs[q].w[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_l, b_off + t * 1024, (pass * kD + q) * tiled::kLChunk, 0);
        __syncthreads();
      }
      const unsigned char* ar = smem + arow * kRowBytes + 64 * lh;
#pragma unroll
      for (int q = 0; q < kD; ++q)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int tm = 0; tm < kMT; ++tm) {
            const h8 af = *reinterpret_cast<const h8*>(ar + tm * 32 * kRowBytes + 128 * q + 16 * t);
            acc2[tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, __builtin_bit_cast(h8, bs[q].w[t]), acc2[tm], 0, 0, 0);
          }
    }
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tm][i] = __builtin_fmaf(g.alpha, acc2[tm][i], acc[tm][i]);
  }

  GLOWQ_STAMP(5);
  // ---- the K groups' accumulators meet in LDS: groups 1.. leave theirs, group 0 adds them in order ---------------
  if constexpr (kWk > 1) {
    __syncthreads();  // every group is done with its stages
    float* red = reinterpret_cast<float*>(smem_all);
    if (gk > 0) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int i = 0; i < 16; ++i) red[((((gk - 1) * cw + wave) * kMT + tm) * 16 + i) * 64 + lane] = acc[tm][i];
    }
    __syncthreads();
    if (gk > 0) return;
#pragma unroll
    for (int o = 1; o < kWk; ++o)
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tm][i] += red[((((o - 1) * cw + wave) * kMT + tm) * 16 + i) * 64 + lane];
  }

  // ---- epilogue: accumulator register i of row tile tm is token row 32 tm + 8 (i / 4) + 4 lh + i % 4, column ln of
  // the wave's row block
  GLOWQ_STAMP(6);
  if (!live) return;
  const int n = rb * 32 + ln;
  if (slices > 1) {
    float* prow = g.partials + ((size_t)blockIdx.y * M) * g.ldp + mem.col0 + n;
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = 32 * tm + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < M) prow[(size_t)m * g.ldp] = acc[tm][i];
      }
    return;
  }
  if (n >= mem.N) return;
  const float bias = mem.bias ? (float)mem.bias[n] : 0.f;
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = 32 * tm + 8 * (i >> 2) + 4 * lh + (i & 3);
      if (m < M) mem.y[(size_t)m * mem.ldy + n] = (half_t)(acc[tm][i] + bias);
    }
}

// y = fp16(sum over the K slices, in slice order, + bias).  One thread per (token row, four columns of the padded row).
__global__ __launch_bounds__(256) void skinny_tiled_reduce_kernel(const TileArgs g) {
  const int c4 = (int)(blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int m = (int)blockIdx.y;
  if (c4 >= g.ldp) return;
  f4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < g.slices; ++s) sum += *reinterpret_cast<const f4*>(g.partials + ((size_t)s * g.M + m) * g.ldp + c4);
  TileMember mem = g.mem[0];
  for (int i = 1; i < g.n_members; ++i)
    if (c4 >= g.mem[i].col0) mem = g.mem[i];
  const int n0 = c4 - mem.col0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int n = n0 + e;
    if (n < mem.N) mem.y[(size_t)m * mem.ldy + n] = (half_t)(sum[e] + (mem.bias ? (float)mem.bias[n] : 0.f));
  }
}

// ---- packing (conversion time) ------------------------------------------------------------------------------
// One thread per (row block, super-block, lane): its four 16-byte pieces; lanes 0..31 also write their column's side pair.
__global__ __launch_bounds__(256) void pack_tiled_weights_kernel(const int32_t* __restrict__ qweight, const half_t* __restrict__ scales,
                                                                 const int32_t* __restrict__ qzeros, unsigned char* __restrict__ out,
                                                                 int N, int K, int group_size, int ldw, int lds, int ldz) {
  const int SB = K >> 8;
  const long total = (long)((N + 31) >> 5) * SB * 64;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int l = (int)(idx & 63);
    const long chunk = idx >> 6;  // = sb * RB + rb
    const int RB = (N + 31) >> 5;
    const int rb = (int)(chunk % RB), sb = (int)(chunk / RB);
    const int row = rb * 32 + (l & 31), h = l >> 5;
    unsigned char* dst = out + (size_t)chunk * tiled::kChunk;
    const bool in = row < N;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (in) {
        const int32_t* src = qweight + (size_t)row * ldw + sb * 32 + 16 * (j >> 1) + 8 * h + 4 * (j & 1);
        v = u32x4{mask_order_word((uint32_t)src[0]), mask_order_word((uint32_t)src[1]), mask_order_word((uint32_t)src[2]),
                  mask_order_word((uint32_t)src[3])};
      }
      *reinterpret_cast<u32x4*>(dst + 1024 * j + 16 * l) = v;
    }
    if (h == 0) {
      u32x2 side = {0u, 0u};
      if (in) {
#pragma unroll
        for (int gh = 0; gh < 2; ++gh) {
          const int grp = (sb * 256 + gh * 128) / group_size;
          const uint32_t z = nibble((uint32_t)qzeros[(size_t)row * ldz + (grp >> 3)], grp & 7);
          const half_t nz = (half_t)(-(float)z * 0x1p-16f);  // a multiple of 2^-24: exact
          side[gh] = (uint32_t)__builtin_bit_cast(uint16_t, scales[(size_t)row * lds + grp]) | ((uint32_t)__builtin_bit_cast(uint16_t, nz) << 16);
        }
      }
      *reinterpret_cast<u32x2*>(dst + tiled::kCodeBytes + 8 * (l & 31)) = side;
    }
  }
}

// One thread per (row block, rank block, lane, k-step): 8 consecutive halves of a row of L, those at positions 2, 3, 6, 7
// times 16.
__global__ __launch_bounds__(256) void pack_tiled_left_kernel(const half_t* __restrict__ L, unsigned char* __restrict__ out, int N,
                                                              int rank) {
  const int LB = (rank + 63) >> 6;
  const long total = (long)((N + 31) >> 5) * LB * 256;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int l = (int)(idx & 63), t = (int)((idx >> 6) & 3);
    const long chunk = idx >> 8;
    const int jb = (int)(chunk % LB), rb = (int)(chunk / LB);
    const int row = rb * 32 + (l & 31), k0 = jb * 64 + (l >> 5) * 32 + t * 8;
    h8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const half_t val = (row < N && k0 + e < rank) ? L[(size_t)row * rank + k0 + e] : (half_t)0.f;
      v[e] = (e & 2) ? val * (half_t)16.f : val;  // the pairs the activations carry divided by 16
    }
    *reinterpret_cast<h8*>(out + (size_t)chunk * tiled::kLChunk + 1024 * t + 16 * l) = v;
  }
}

// ---- host side ----------------------------------------------------------------------------------------------
#if GLOWQ_TDBG & 32
extern "C" int glowq_debug_stamps(void* host, size_t bytes, int clear) {
  if (clear) { void* p; hipGetSymbolAddress(&p, HIP_SYMBOL(g_tstamps)); return (int)hipMemset(p, 0, sizeof(g_tstamps)); }
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tstamps), bytes < sizeof(g_tstamps) ? bytes : sizeof(g_tstamps));
}
#endif
hipError_t launch_pack_tiled(const int32_t* qweight, const half_t* scales, const int32_t* qzeros, void* out, int N, int K,
                             int group_size, int ldw, int lds, int ldz, int num_cus, hipStream_t stream) {
  const long total = (long)((N + 31) >> 5) * (K >> 8) * 64;
  long blocks = (total + 255) / 256;
  if (blocks > (long)num_cus * 32) blocks = (long)num_cus * 32;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(pack_tiled_weights_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, qweight, scales, qzeros,
                     static_cast<unsigned char*>(out), N, K, group_size, ldw, lds, ldz);
  return hipGetLastError();
}

hipError_t launch_pack_tiled_left(const half_t* L, void* out, int N, int rank, int num_cus, hipStream_t stream) {
  const long total = (long)((N + 31) >> 5) * ((rank + 63) >> 6) * 256;
  long blocks = (total + 255) / 256;
  if (blocks > (long)num_cus * 32) blocks = (long)num_cus * 32;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(pack_tiled_left_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, L, static_cast<unsigned char*>(out), N, rank);
  return hipGetLastError();
}

// Every member brings its tiled weights (and its tiled left factor where it has one), K and the groups fit the layout,
// the rank is a multiple of 8 and at most 64 token rows.
bool skinny_tiled_supported(const GroupDev& g) {
  if (g.M < 1 || g.M > 64 || !tiled::applies(g.K, g.group_size)) return false;
  const half_t* r = g.r != nullptr ? g.r : (g.R != nullptr ? g.r_out : nullptr);
  if (r != nullptr && ((g.rank & 7) != 0 || g.rank < 8 || (reinterpret_cast<uintptr_t>(r) & 15u) != 0)) return false;
  if ((reinterpret_cast<uintptr_t>(g.x) & 15u) != 0) return false;
  if ((size_t)g.M * g.K * 2 >= (1ull << 32)) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if (m.tiled == nullptr || (reinterpret_cast<uintptr_t>(m.tiled) & 15u) != 0) return false;
    if (tiled::weight_bytes(m.N, g.K) >= (1ull << 32)) return false;  // 32-bit offsets into the stream
    if (m.L != nullptr && r != nullptr && (m.tiled_L == nullptr || m.tiled_rank != g.rank || (reinterpret_cast<uintptr_t>(m.tiled_L) & 15u) != 0))
      return false;
  }
  return true;
}

// How the launch cuts K and staffs a K group: `wk` K groups inside a workgroup (their sums meet in LDS), `slices`
// workgroups per tile (their sums meet in the workspace), `pw` producer waves per K group.  A SIMD wants two waves and
// more (a lone wave issues most vector instructions at half rate), so two K groups wherever K has the depth; slices
// where the tiles alone leave most of the chip empty.  Workgroups stay at 768 threads and below (a 1024-thread
// workgroup gets 128 registers per lane and the chip runs such workgroups in two rounds).
struct TiledPlan {
  int wk, slices, pw, cw;
};
static int tiled_tiles(const GroupDev& g, int cw) {
  int t = 0;
  for (int i = 0; i < g.n_members; ++i) t += ((g.mem[i].N + 31) / 32 + cw - 1) / cw;
  return t;
}
static TiledPlan tiled_plan(const GroupDev& g, int num_cus, size_t ws_bytes) {
  static const int env_slices = getenv("GLOWQ_TILED_SLICES") ? atoi(getenv("GLOWQ_TILED_SLICES")) : 0;
  static const int env_wk = getenv("GLOWQ_TILED_WK") ? atoi(getenv("GLOWQ_TILED_WK")) : 0;
  static const int env_pw = getenv("GLOWQ_TILED_PW") ? atoi(getenv("GLOWQ_TILED_PW")) : 0;
  static const int env_cw = getenv("GLOWQ_TILED_CW") ? atoi(getenv("GLOWQ_TILED_CW")) : 0;
  const int SB = g.K >> 8;
  TiledPlan p{1, 1, 1, 4};
  // a few tiles more than compute units would run as two rounds, the second nearly empty: wider tiles (one K group)
  // where they bring the count down to one round
  if (tiled_tiles(g, 4) > num_cus) {
    for (int cw = 5; cw <= (g.M <= 32 ? 8 : 6); ++cw)
      if (tiled_tiles(g, cw) <= num_cus) {
        p.cw = cw;
        break;
      }
  }
  if (env_cw >= 1 && env_cw <= (g.M <= 32 ? 8 : 6)) p.cw = env_cw;
  // two K groups: up to 16 token rows on tiles that fill the chip by themselves (more rows want four producer waves, and
  // a K range cut into slices is short enough already).  8B shapes, launch with the projection, us, two groups / one:
  // gate|up 8 rows 22.4 / 24.1, 32 rows 26.4 / 26.3; down_proj 32 rows 27.1 / 25.5
  int wk = (SB >= 8 && p.cw <= 4 && g.M <= 16 && tiled_tiles(g, p.cw) * 2 > num_cus) ? 2 : 1;
  if (env_wk == 1 || (env_wk == 2 && p.cw <= 4 && g.M <= 32)) wk = env_wk;
  p.pw = g.M <= 8 ? 1 : (g.M <= 16 || wk == 2 ? 2 : 4);
  // two row tiles per wave: 512 threads, their registers allow no more -- four producer waves beside four consumers, three
  // beside five, two beside six
  if (g.M > 32) wk = 1, p.pw = p.cw > 5 ? 2 : (p.cw > 4 ? 3 : 4);
  if (env_pw == 2 && g.M > 8) p.pw = 2;
  if (env_pw == 3 && g.M > 32 && p.cw <= 5) p.pw = 3;
  if (env_pw == 4 && g.M > 16 && wk == 1 && (g.M <= 32 || p.cw <= 4)) p.pw = 4;
  p.wk = wk;
  const int tiles = tiled_tiles(g, p.cw);
  long ldp = 0;
  for (int i = 0; i < g.n_members; ++i) ldp += ((g.mem[i].N + 31) / 32 + p.cw - 1) / p.cw * p.cw * 32;
  long s = env_slices > 0 ? env_slices : (tiles * 2 <= num_cus ? num_cus / tiles : 1);
  if (s > SB / (4 * wk)) s = SB / (4 * wk);
  const size_t per_slice = (size_t)g.M * ldp * sizeof(float);
  if (per_slice > 0 && (size_t)s > ws_bytes / per_slice) s = (long)(ws_bytes / per_slice);
  if (s < 1) s = 1;
  const int per = (SB + (int)s - 1) / (int)s;  // slices of equal depth: no more of them than leave none empty
  p.slices = (SB + per - 1) / per;
  return p;
}

// The most workspace tiled_plan asks for: it cuts K only where tiles x slices stay within num_cus workgroups, and such
// groups have tiles of four consumer waves (128 columns): one 128-column fp32 tile per token row for each of them.
size_t tiled_split_workspace_bytes(int M, int num_cus) { return M > 4 ? (size_t)num_cus * (size_t)M * 128 * sizeof(float) : 0; }

template <int kRows, int kWk, int kPW, bool kProj = false>
static hipError_t launch_tiled_t(TileArgs& a, const half_t* x, int num_cus, hipStream_t stream) {
  auto kern = skinny_tiled_kernel<kRows, kWk, kPW, kProj>;
  constexpr int kMT = kRows > 32 ? 2 : 1;
  size_t lds = (size_t)kWk * 2 * (kRows * kRowBytes + 2 * kRows * 16);
  const size_t red = (size_t)(kWk - 1) * a.cw * kMT * 16 * 64 * sizeof(float);
  if (lds < red) lds = red;
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
  if (a.cw < 1 || a.cw > tiled_max_cw(kRows, kWk, kPW)) return hipErrorInvalidValue;
  const int threads = (a.cw + kPW) * 64 * kWk;
  int grid_x = a.tiles;
  if constexpr (kProj) {
    // The workgroups in front take places the launch leaves free on the chip, so that every workgroup starts at once and
    // none with a column tile waits behind a producer.  The readers ask for r during their last super-block, so a
    // producer has most of the launch for its blocks: up to `per_producer` of them (GLOWQ_TILED_PROJ_BLOCKS).
    static std::atomic<long> asked_for{-1};
    static std::atomic<int> resident{0};
    const long shape = (long)lds * 4096 + threads;
    int per_cu = 0;
    if (asked_for.load(std::memory_order_acquire) == shape) {
      per_cu = resident.load(std::memory_order_relaxed);
    } else {
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), threads, lds) != hipSuccess) per_cu = 0;
      resident.store(per_cu, std::memory_order_relaxed);
      asked_for.store(shape, std::memory_order_release);
    }
    static const int env_blocks = getenv("GLOWQ_TILED_PROJ_BLOCKS") ? atoi(getenv("GLOWQ_TILED_PROJ_BLOCKS")) : 0;
    static const int env_producers = getenv("GLOWQ_TILED_PRODUCERS") ? atoi(getenv("GLOWQ_TILED_PRODUCERS")) : 0;
    const int per_producer = env_blocks > 0 ? env_blocks : kTiledProjBlocks;
    // (one workgroup per compute unit, whatever the occupancy allows: two that share a compute unit share its LDS
    // bandwidth and matrix cores, and the launch gets longer -- gate|up of a 14B layer at eight rows with 131 producers
    // beside 218 tiles 42 us against 30.5)
    const long capacity = per_cu >= 1 ? num_cus : 0;
    long want = (capacity - (long)a.tiles) & ~3L;  // (the front is padded to a multiple of four: handover.hpp)
    if (env_producers > 0) want = env_producers;
    const int nblocks = ((a.rank + 3) / 4) * ((a.M + 3) / 4);  // blocks of r: four token rows by four rows of R
    if (want > nblocks) want = nblocks;
    if (want > kTiledMaxProducers) want = kTiledMaxProducers;
    if (threads < 256 || want < 1 || ((long)per_producer * want < nblocks && a.spin != 0xFFFFFFFFu)) return hipErrorNotReady;
    a.producers = (int)want;
    a.teams = (nblocks > want && threads >= 512) ? 2 : 1;  // two blocks at a time where the workgroup has the waves
    grid_x = front_grid(a.tiles, a.producers);
  }
  hipLaunchKernelGGL(kern, dim3(grid_x, a.slices), dim3(threads), lds, stream, x, a.M, a.K, a.slices, a.mem[0].wt,
                     a.blk_end[0], a.mem[0].N, a.cw, a);
  note_launch(grid_x, a.slices, threads, kProj ? "skinny_tiled_kernel<%d,%d,%d,1> with %d consumer waves" : "skinny_tiled_kernel<%d,%d,%d> with %d consumer waves",
              kRows, kWk, kPW, a.cw);
  if (hipError_t e = hipGetLastError(); e != hipSuccess || a.slices == 1) return e;
  hipLaunchKernelGGL(skinny_tiled_reduce_kernel, dim3((a.ldp / 4 + 255) / 256, a.M), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_skinny_tiled(GroupDev& g, int num_cus, hipStream_t stream) {
  TileArgs a;
  a.r = g.r;
  // the launch computes r itself (run_group set g.pub to the head of the workspace): up to 16 token rows and rank 256 (r
  // goes through the stages in one pass), K whole, nothing else in the workspace (no slices)
  const bool proj = g.pub != nullptr;
  a.R = g.R;
  a.r_out = g.r_out;
  a.pub = g.pub;
  a.spin = g.pub_mute ? 0xFFFFFFFFu : g.pub_spin;
  a.producers = 0;
  a.teams = 1;
  if (proj) {
    if (g.M > 16 || g.rank > 256 || (g.rank & 7) != 0 || (g.K & 7) != 0 || g.R == nullptr || g.r_out == nullptr || g.ws_bytes < kTiledHandoverBytes)
      return hipErrorNotReady;
    a.r = g.r_out;
  }
  a.n_members = g.n_members;
  a.M = g.M;
  a.K = g.K;
  a.rank = g.rank;
  a.alpha = g.alpha;
  const bool ws_ok = g.ws != nullptr && (reinterpret_cast<uintptr_t>(g.ws) & 15u) == 0;
  a.partials = ws_ok ? static_cast<float*>(g.ws) : nullptr;
  const TiledPlan plan = tiled_plan(g, num_cus, ws_ok ? g.ws_bytes : 0);
  a.slices = plan.slices;
  a.cw = plan.cw;
  int tiles = 0, col = 0;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    TileMember& t = a.mem[i];
    t.wt = static_cast<const unsigned char*>(m.tiled);
    t.lt = (m.L != nullptr && (g.r != nullptr || proj)) ? static_cast<const unsigned char*>(m.tiled_L) : nullptr;
    t.bias = m.bias;
    t.y = m.y;
    t.N = m.N;
    t.ldy = m.ldy;
    t.col0 = col;
    const int mt = ((m.N + 31) / 32 + plan.cw - 1) / plan.cw;
    tiles += mt;
    col += mt * plan.cw * 32;
    a.blk_end[i] = tiles;
  }
  a.tiles = tiles;
  a.ldp = col;
  const int key = (g.M <= 8 ? 8 : g.M <= 16 ? 16 : g.M <= 32 ? 32 : 64) * 100 + plan.wk * 10 + plan.pw;
  if (proj) {
    if (a.slices != 1) return hipErrorNotReady;
    switch (key) {
      case 821: return launch_tiled_t<8, 2, 1, true>(a, g.x, num_cus, stream);
      case 811: return launch_tiled_t<8, 1, 1, true>(a, g.x, num_cus, stream);
      case 1622: return launch_tiled_t<16, 2, 2, true>(a, g.x, num_cus, stream);
      case 1612: return launch_tiled_t<16, 1, 2, true>(a, g.x, num_cus, stream);
    }
    return hipErrorNotReady;
  }
  switch (key) {
    case 821: return launch_tiled_t<8, 2, 1>(a, g.x, num_cus, stream);
    case 811: return launch_tiled_t<8, 1, 1>(a, g.x, num_cus, stream);
    case 1622: return launch_tiled_t<16, 2, 2>(a, g.x, num_cus, stream);
    case 1612: return launch_tiled_t<16, 1, 2>(a, g.x, num_cus, stream);
    case 3222: return launch_tiled_t<32, 2, 2>(a, g.x, num_cus, stream);
    case 3212: return launch_tiled_t<32, 1, 2>(a, g.x, num_cus, stream);
    case 3214: return launch_tiled_t<32, 1, 4>(a, g.x, num_cus, stream);
    case 6412: return launch_tiled_t<64, 1, 2>(a, g.x, num_cus, stream);
    case 6413: return launch_tiled_t<64, 1, 3>(a, g.x, num_cus, stream);
    case 6414: return launch_tiled_t<64, 1, 4>(a, g.x, num_cus, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace glowq
