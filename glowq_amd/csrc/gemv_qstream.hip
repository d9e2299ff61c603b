// Decode GEMV for 2..4 token rows: the arithmetic of the 4x4x4 matrix-core GEMV (gemv_quad.hip) under the memory
// schedule of the stream GEMV (stream_kernel.hpp).
//
// v_mfma_f32_4x4x4_16B_f16 multiplies sixteen independent 4x4x4 blocks: lanes 4b..4b+3 form block b, lane 4b + q
// supplies four k values of row q of A and of column q of B and receives column q of the result.  Row q of A is token
// row q of the activations, column q of B is an output row of the weights, so one instruction pair per 8 codes serves
// four token rows.  The codes are used in place as fp16 subnormals, the zero-point is folded through per-unit
// activation sums, the correction rides along as a K-extension with the rows of L as B operands (gemv_quad.hip).
//
// A wave takes a tile of 8 output rows (two row blocks of four) by 64 units of 32 columns -- or 16 rows by 32 units --
// and issues every load of it at its head, right behind the loads of the activations; it then stages the activations,
// meets the other waves at the barrier, and consumes the weights in the order they return, each 16-byte word behind a
// wait that counts exactly the loads issued after it.  The loads are inline assembly for that reason, are never under a
// condition (a wave or a lane without work reads an address that is valid anyway), and the kernel must compile without
// scratch memory.
//
// What bounds this kernel next to memory is the LDS pipe and the vector ALU, and the tile is shaped for them:
//   * the A operands (the activations of 16 units, 16 bytes per lane and word) are read from LDS once per 16-unit
//     column of the tile and serve its row blocks from registers;
//   * the weights are loaded in the layout the matrix core wants -- lane 4b + q reads unit b of row q of a row block:
//     a load covers 256 contiguous bytes of each of four rows -- so no lane exchange lies between load and use
//     (with loads in memory order and a ds_bpermute per dword the LDS pipe was busy 80 % of the launch);
//   * the activations of the upper nibbles are staged divided by 16, so one accumulator chain takes both nibbles;
//   * the waves that share the rows of a tile (the slices of their K extent) meet in LDS once per tile, at its end;
//   * a workgroup is one or two tiles wide: small workgroups come and go independently, which is worth more than the
//     activation rows they stage redundantly;
//   * a launch of more workgroups than the compute units hold at once runs as many as they hold, each walking a list
//     of tiles: the activations are staged once, and a wave's next requests go out as soon as its last tile is stored.
#include <cstdlib>

#include "stream_kernel.hpp"

namespace glowq {

using namespace streamk;

namespace {

// A wave's tile: kR row blocks of four rows by kC columns of 16 units, eight 16-byte loads per lane either way:
// 8 rows by 2048 columns (kR = 2) or 16 rows by 1024 columns (kR = 4; with eight token rows, two sets of sums per row
// block, that one does not fit the 128 registers a wave of a 16-wave workgroup has).
__host__ __device__ constexpr int qs_c(int r) { return 8 / r; }
constexpr int kQsPad = 4;          // 16-byte words between the token rows of xs beyond 4 U: spreads the four tokens of a
                                   // block over the banks (1, 2 and 4 measured: 19.0, 17.1, 16.6 us on 28672 x 4096)

// xs   [tokens][4 U + kQsPad] of 8 halves: word t of unit u of token m at m * x_stride + t * U + u, holding
//      x[32u + 8t + {0,4,2,6, 1,5,3,7}] (the order the two masked operands of a code word come out in)
// sig  [U][tok4] floats: 2^-24 * sum of the 32 activations of unit u, per token
// rs   [tok4][rank + 8] halves
// part [2][waves][kR][sets][4 rows of lanes][4 rows][4 tokens] floats: what the waves leave for the final sum (two
//      buffers, used in turn by the tiles a workgroup walks)
struct QsLds {
  int tok4, x_stride, r_stride;
  size_t sig_off, r_off, part_off, total;
};
__host__ __device__ inline QsLds qs_lds(int tokens, int K, int rank, int waves, int r) {
  QsLds l;
  const int U = K >> 5;
  l.tok4 = (tokens + 3) & ~3;
  l.x_stride = 4 * U + kQsPad;
  l.r_stride = rank + 8;
  l.sig_off = (size_t)tokens * l.x_stride * 16;
  l.r_off = l.sig_off + (size_t)U * l.tok4 * sizeof(float);
  l.part_off = l.r_off + (rank > 0 ? (size_t)l.tok4 * l.r_stride * sizeof(half_t) : 0);
  l.total = l.part_off + (size_t)2 * waves * r * (l.tok4 / 4) * 64 * sizeof(float);
  return l;
}

// sum over the 4 lanes of a row of 16 lanes that share lane % 4; every lane gets the total of its class
__device__ __forceinline__ float row_class_sum(float v) {
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true);  // row_ror:4
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true);  // row_ror:8
  v += __builtin_bit_cast(float, t);
  return v;
}

// kR: row blocks of a wave's tile (2 or 4; kC = 8 / kR columns of 16 units); kLD: dwords of a row of L per lane (0, 4
// or 8: sixteen lanes cover rank <= 32 kLD); kTok: token rows staged (2, 4 or 8); kXW: 16-byte words of each token row per thread.  `slices` = ceil(K / (512 kC)) consecutive waves of a workgroup
// share the rows of a tile, slice s taking units 16 kC s ... 16 kC (s + 1) - 1 (units past the row read its last unit
// again and are weighted by zero).
template <int kR, int kLD, int kTok, int kXW>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(2, 4)))
void gemv_qstream_kernel(const GroupDev g, const int slices, const int tiles_per_wg, const int total_wgs) {
  constexpr int kC = qs_c(kR), kRows = 4 * kR;
  constexpr int kSets = (kTok + 3) / 4;
  constexpr int kTok4 = 4 * kSets;
  constexpr int kLast = kTok - 4 * (kSets - 1);  // token rows of the last set that are worth finishing
  constexpr int kLQ = kLD / 4;                   // 16-byte loads of a row of L per lane
  constexpr int kGmax = 4 * kC;                  // groups of a tile row at 128 columns per group
  constexpr int kSideLoads = kR * kC / 4;        // (row, group) pairs of a tile / 64 lanes
  constexpr int kWeights = kR * kC;              // weight loads of the tile
  constexpr int kLoads = 2 * kSideLoads + kR * kLQ + kWeights;
  static_assert(kTok * kXW + kTok4 + kLoads <= 63, "vmcnt is a 6-bit field");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = g.K, U = K >> 5, rank = g.rank;
  const int upg_shift = __builtin_ctz(g.group_size >> 5);
  const int G = (U + (1 << upg_shift) - 1) >> upg_shift;
  const int threads = blockDim.x, waves = threads >> 6;
  const QsLds lay = qs_lds(kTok, K, kLD > 0 ? rank : 0, waves, kR);
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + lay.sig_off);
  half_t* rs = reinterpret_cast<half_t*>(smem + lay.r_off);
  float* part = reinterpret_cast<float*>(smem + lay.part_off);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int qb = lane >> 2, qj = lane & 3;  // block and column of the matrix-core layout

  // ---- activations first: their wait then does not cover the weight requests issued behind them
  const int words = K >> 3, rd = rank >> 1;
  u32x4 xw[kTok][kXW];
  uint32_t rw[kLD > 0 ? kTok4 : 1];
#pragma unroll
  for (int m = 0; m < kTok; ++m) {
    const half_t* xrow = g.x + (size_t)min(m, g.M - 1) * K;  // token rows past M repeat row M - 1 and are never stored
#pragma unroll
    for (int i = 0; i < kXW; ++i) xw[m][i] = ld_b128(xrow, (uint32_t)min((int)threadIdx.x + i * threads, words - 1) * 16u);
  }
  if constexpr (kLD > 0) {
#pragma unroll
    for (int m = 0; m < kTok4; ++m)
      rw[m] = ld_b32(g.r + (size_t)min(m, g.M - 1) * rank, (uint32_t)min((int)threadIdx.x, rd - 1) * 4u);
  }

  // ---- the wave's place in its workgroup (tiles_per_wg is 1..4: three comparisons instead of a division)
  const int local_tile = (wave >= slices) + (wave >= 2 * slices) + (wave >= 3 * slices);
  const int slice = wave - local_tile * slices;
  const int unit0 = slice * (16 * kC);  // first unit of the slice
  const int grp0 = unit0 >> upg_shift;  // and its group
  const int l_chunks = kLD > 0 ? rank / (2 * kLD) : 1;  // lanes of a row that hold a part of L

  // ---- what a wave holds of a tile: set by issue(), used by finish()
  MemberDev mem = g.mem[0];
  bool valid = false, l_here = false;
  int row0 = 0;
  uint32_t sc[kSideLoads], zw[kSideLoads], sgrp[kSideLoads];
  u32x4 lq[kLQ > 0 ? kR : 1][kLQ > 0 ? kLQ : 1];
  u32x4 w[kC][kR];

  // The launch is a list of total_wgs workgroups' worth of tiles (per member: its tiles in sets of tiles_per_wg); the
  // workgroups that run take them round robin, vwg = blockIdx.x, blockIdx.x + gridDim.x, ...  A launch with more of
  // them than the compute units hold at once runs that many workgroups and lets each walk its list: the activations
  // are staged once, and a wave requests its next tile the moment it has stored the last one.
  auto issue = [&](const int vwg) {
  // ---- member and tile of this wave
  mem = g.mem[0];
  int wg_begin = 0, total_tiles = g.task_end[0];
#define GLOWQ_PICK(i)                                  \
  if (g.n_members > i && vwg >= g.wg_end[i - 1]) {    \
    mem = g.mem[i];                                    \
    wg_begin = g.wg_end[i - 1];                        \
    total_tiles = g.task_end[i] - g.task_end[i - 1];   \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int want = (vwg - wg_begin) * tiles_per_wg + local_tile;
  // waves past the member's last tile (and the waves a workgroup has beyond whole sets of slices) still issue their
  // loads (the wait counts stay what they are), all lanes on one address
  valid = want < total_tiles && local_tile < tiles_per_wg;
  row0 = (valid ? want : 0) * kRows;
  const uint32_t live = valid ? 0xFFFFFFFFu : 0u;
  // Every member's buffers stay below 2 GiB (checked on the host): uniform base + 32-bit byte offset, row index and
  // row pitch below 2^24 each.  (24-bit multiplies: the 32-bit multiply-add this compiler would otherwise pick takes a
  // register pair as its addend, with whatever register lies next to the addend as the unused upper half -- possibly
  // one a load is still writing.)
  const uint32_t ldw_bytes = (uint32_t)mem.ldw * 4u, lds_bytes = (uint32_t)mem.lds * 2u, ldz_bytes = (uint32_t)mem.ldz * 4u;

  // ---- every load of the tile
  // scale and zero-point word of one (row, group) pair per lane and load: pair p = 64 j + lane is group p % kGmax of the
  // slice, row p / kGmax of the tile
#pragma unroll
  for (int j = 0; j < kSideLoads; ++j) {
    const int p = 64 * j + lane;
    const uint32_t n = (uint32_t)min(row0 + p / kGmax, mem.N - 1);
    sgrp[j] = (uint32_t)min(grp0 + p % kGmax, G - 1);
    sc[j] = ld_u16_nt(mem.scales, (__umul24(n, lds_bytes) + sgrp[j] * 2u) & live);
    zw[j] = ld_b32_nt(mem.qzeros, (__umul24(n, ldz_bytes) + (sgrp[j] >> 3) * 4u) & live);
  }
  uint32_t n_q[kR];  // the lane's row of each row block
#pragma unroll
  for (int rb = 0; rb < kR; ++rb) n_q[rb] = (uint32_t)min(row0 + 4 * rb + qj, mem.N - 1);
  // the last slice, the one with the fewest columns left, adds the correction
  l_here = kLD > 0 && mem.L != nullptr && slice == slices - 1;
  if constexpr (kLD > 0) {
    // elsewhere: valid memory, weighted by zero
    const char* lb = l_here ? reinterpret_cast<const char*>(mem.L) : reinterpret_cast<const char*>(g.x);
#pragma unroll
    for (int rb = 0; rb < kR; ++rb) {
      const uint32_t lo = l_here ? ((__umul24(n_q[rb], (uint32_t)rank * 2u) + (uint32_t)min(qb, l_chunks - 1) * (4u * kLD)) & live) : 0u;
#pragma unroll
      for (int j = 0; j < kLQ; ++j) lq[rb][j] = ld_b128_nt(lb + 16 * j, lo);
    }
  }
#pragma unroll
  for (int c = 0; c < kC; ++c) {
    const uint32_t u = (uint32_t)min(unit0 + 16 * c + qb, U - 1);
#pragma unroll
    for (int rb = 0; rb < kR; ++rb) w[c][rb] = ld_b128_nt(mem.qweight, (__umul24(n_q[rb], ldw_bytes) + u * 16u) & live);
  }
  };  // issue()
  issue((int)blockIdx.x);

  // ---- stage the activations (every load of x and r lies ahead of the tile's: one count covers them all)
#pragma unroll
  for (int m = 0; m < kTok; ++m) {
    wait_words<kLoads>(xw[m]);
#pragma unroll
    for (int i = 0; i < kXW; ++i) {
      if (i * threads >= words) break;  // uniform: the words of this round lie past the row for every thread
      const int wd = (int)threadIdx.x + i * threads;
      const h8 v = __builtin_bit_cast(h8, xw[m][i]);
      const h2 ones = {(half_t)1.f, (half_t)1.f};
      float s = __builtin_amdgcn_fdot2(h2{v[0], v[1]}, ones, 0.f, false);
      s = __builtin_amdgcn_fdot2(h2{v[2], v[3]}, ones, s, false);
      s = __builtin_amdgcn_fdot2(h2{v[4], v[5]}, ones, s, false);
      s = __builtin_amdgcn_fdot2(h2{v[6], v[7]}, ones, s, false);
      s = quad_sum(s);  // threads and words are multiples of 4: a quad lies inside the row or outside as a whole
      if (wd < words) {
        h8 p;
        p[0] = v[0]; p[1] = v[4]; p[2] = v[2]; p[3] = v[6];
        // the upper nibbles come out of the mask as code * 2^-20: their activations carry the 1/16 (exact but for
        // values below 2^-10, which lose bits worth 2^-25 and less)
        const half_t sixteenth = (half_t)0.0625f;
        p[4] = v[1] * sixteenth; p[5] = v[5] * sixteenth; p[6] = v[3] * sixteenth; p[7] = v[7] * sixteenth;
        const int u = wd >> 2, t = wd & 3;
        xs[(size_t)m * lay.x_stride + t * U + u] = p;
        if (t == 0) sig[u * kTok4 + m] = s * 0x1p-24f;
      }
    }
  }
  if constexpr (kLD > 0) {
#pragma unroll
    for (int m = 0; m < kTok4; ++m) {
      wait_vm<kLoads>(rw[m]);
      if ((int)threadIdx.x < rd) reinterpret_cast<uint32_t*>(rs + m * lay.r_stride)[threadIdx.x] = rw[m];
    }
  }
  __syncthreads();

  // ---- consume the tile in the order it was requested, then reduce and store it.  `parity` picks one of the two
  // buffers the waves leave their sums in: the sums of one tile are read while those of the next may be written.
  auto finish = [&](const int parity) {
  f4 tot[kR][kSets];
#pragma unroll
  for (int rb = 0; rb < kR; ++rb)
#pragma unroll
    for (int s = 0; s < kSets; ++s) tot[rb][s] = f4{0.f, 0.f, 0.f, 0.f};
  // the side loads sit ahead of the weights: the same count covers them.  Scale bits and zero-point of the pair a lane
  // loaded are packed for the lane exchange.
  uint32_t side[kSideLoads];
#pragma unroll
  for (int j = 0; j < kSideLoads; ++j) {
    wait_vm<kWeights>(sc[j]);
    wait_vm<kWeights>(zw[j]);
    side[j] = (sc[j] & 0xFFFFu) | (nibble(zw[j], (int)(sgrp[j] & 7u)) << 16);
  }
  if constexpr (kLD > 0) {
    // the correction first: tot = alpha 2^-24 (L r), the accumulators carry 2^-24
    const bool l_live = l_here && qb < l_chunks;
    const int chunk = min(qb, l_chunks - 1);
    const float alpha_scaled = g.alpha * 0x1p-24f;
    h4 ra[kSets][2 * kLQ];
#pragma unroll
    for (int s = 0; s < kSets; ++s) {
      const int tok = (kTok >= 4) ? 4 * s + qj : min(qj, kTok - 1);
      const half_t* rt = rs + tok * lay.r_stride + chunk * (2 * kLD);
#pragma unroll
      for (int j = 0; j < 2 * kLQ; ++j) ra[s][j] = *reinterpret_cast<const h4*>(rt + 4 * j);
    }
#pragma unroll
    for (int rb = 0; rb < kR; ++rb) {
#pragma unroll
      for (int j = 0; j < kLQ; ++j) wait_vm<kWeights>(lq[rb][j]);
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 2 * kLQ; ++j) {
          const u32x2 bw = {l_live ? lq[rb][j >> 1][2 * (j & 1)] : 0u, l_live ? lq[rb][j >> 1][2 * (j & 1) + 1] : 0u};
          acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ra[s][j], __builtin_bit_cast(h4, bw), acc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) tot[rb][s][i] = alpha_scaled * acc[i];
      }
    }
  }
  static_for<kC>([&](auto CC) {
    constexpr int c = decltype(CC)::value;
    const int uraw = unit0 + 16 * c + qb;
    const bool active = uraw < U;
    int u = active ? uraw : U - 1;
    // the activations of this column of the tile: read once, used by every row block
    wait_vm<(kC - 1 - c) * kR + (kR - 1)>(w[c][0], u);
    const int gi = ((u >> upg_shift) - grp0) & (kGmax - 1);  // group of this unit within the slice
    // One set of four token rows after the other: its activations are read once and serve every row block from
    // registers (both sets at once would not fit the 128 registers a wave of a 16-wave workgroup has).
    uint32_t sv[kR];
#pragma unroll
    for (int s = 0; s < kSets; ++s) {
      const int tok = (kTok >= 4) ? 4 * s + qj : min(qj, kTok - 1);
      const h8* xt = xs + (size_t)tok * lay.x_stride + u;
      h4 a_lo[4], a_hi[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const h8 xv = xt[t * U];
        a_lo[t] = h4{xv[0], xv[1], xv[2], xv[3]};
        a_hi[t] = h4{xv[4], xv[5], xv[6], xv[7]};
      }
      const f4 sg = *reinterpret_cast<const f4*>(sig + u * kTok4 + 4 * s);
      static_for<kR>([&](auto RB) {
        constexpr int rb = decltype(RB)::value;
        constexpr int kBehind = (kC - 1 - c) * kR + (kR - 1 - rb);  // loads issued behind this word
        if (s == 0) {  // (a constant once the loop over the sets is unrolled)
          if constexpr (rb > 0) wait_vm<kBehind>(w[c][rb]);
          // pair (row 4 rb + qj, group gi) was loaded by lane p % 64 of load p / 64 (a constant per row block)
          constexpr int kPair0 = 4 * rb * kGmax;
          sv[rb] = (uint32_t)__builtin_amdgcn_ds_bpermute(((kPair0 & 63) + qj * kGmax + gi) << 2, (int)side[kPair0 >> 6]);
        }
        const float scl = active ? (float)__builtin_bit_cast(half_t, (uint16_t)(sv[rb] & 0xFFFFu)) : 0.f;
        const float zp = (float)(sv[rb] >> 16);
        f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t wd = w[c][rb][t], hi = wd >> 8;
          const h4 b_lo = __builtin_bit_cast(h4, u32x2{wd & 0x000F000Fu, hi & 0x000F000Fu});  // codes 0,4,2,6 * 2^-24
          const h4 b_hi = __builtin_bit_cast(h4, u32x2{wd & 0x00F000F0u, hi & 0x00F000F0u});  // codes 1,5,3,7 * 2^-20
          acc = __builtin_amdgcn_mfma_f32_4x4x4f16(a_lo[t], b_lo, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_4x4x4f16(a_hi[t], b_hi, acc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (s == kSets - 1 && i >= kLast) break;
          tot[rb][s][i] = __builtin_fmaf(scl, __builtin_fmaf(-zp, sg[i], acc[i]), tot[rb][s][i]);
        }
        // The sums are pinned here (an empty statement that "rewrites" them): left alone, the compiler sinks the
        // arithmetic of every word behind the last wait and keeps every loaded word live until then.
        asm volatile("" : "+v"(tot[rb][s]));
      });
    }
  });

  // ---- the 16 lanes of a row: four blocks per row of 16 lanes meet through lane rotations, the four rows of lanes and
  // the slices of the tile through LDS
  {
    float* mine = part + (size_t)(parity * waves + wave) * (kR * kSets * 64);
#pragma unroll
    for (int rb = 0; rb < kR; ++rb) {
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        const f4 v = {row_class_sum(tot[rb][s][0]), row_class_sum(tot[rb][s][1]), row_class_sum(tot[rb][s][2]),
                      row_class_sum(tot[rb][s][3])};
        if ((lane & 12) == 0)  // block 0 of each row of lanes: [rb][s][row of lanes][qj] x 4 tokens
          *reinterpret_cast<f4*>(mine + (((rb * kSets + s) * 4 + (lane >> 4)) * 4 + qj) * 4) = v;
      }
    }
  }
  __syncthreads();  // every wave of the workgroup arrives here once
  if (slice == 0 && valid) {
    // lane = 4 (row of the tile) + token of a set
    const int rowi = min(lane >> 2, kRows - 1), i = lane & 3;
    const int n = row0 + rowi;
    const bool writer = (lane >> 2) < kRows && n < mem.N;
    const float bias = (writer && mem.bias) ? (float)mem.bias[n] : 0.f;
#pragma unroll
    for (int s = 0; s < kSets; ++s) {
      const float* src = part + (size_t)(parity * waves + wave) * (kR * kSets * 64) + ((((rowi >> 2) * kSets + s) * 4) * 4 + (rowi & 3)) * 4 + i;
      float v = 0.f;
      for (int o = 0; o < slices; ++o)
#pragma unroll
        for (int lr = 0; lr < 4; ++lr) v += src[(size_t)o * (kR * kSets * 64) + lr * 16];
      const int m = 4 * s + i;
      if (writer && m < g.M) mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(v, 0x1p24f, bias));
    }
  }
  };  // finish()
  finish(0);
  // the rest of this workgroup's list (the same for all its waves: the barriers inside stay matched)
  int parity = 1;
  for (int vwg = (int)blockIdx.x + (int)gridDim.x; vwg < total_wgs; vwg += (int)gridDim.x) {
    issue(vwg);
    finish(parity);
    parity ^= 1;
  }
}

int qs_env(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

// How a shape is launched: slices per tile, waves per workgroup, words of a token row per
// thread, token rows staged.
struct QsPlan {
  int r, slices, waves, xw, tok, num_cus;
  size_t lds;
};

// tiles_per_wg: 0 for the least that makes a workgroup, else that many (1..4)
bool qs_plan(int M, int K, int rank, bool has_r, int tiles_per_wg, QsPlan& p) {
  static const int env_waves = qs_env("GLOWQ_QSTREAM_WAVES", 0);
  if (M < 2 || M > 4) return false;
  const int U = K >> 5;
  p.tok = M <= 2 ? 2 : 4;
  // Tile: 8 rows by 2048 columns (8B-shape layer at four token rows, 8 x 2048 / 16 x 1024: q|k|v 6.6 / 6.9 us, o_proj
  // 4.7 / 5.0, gate|up 15.9 / 16.8, down_proj 11.5 / 12.3; K = 5120, 2.5 slices of 2048 columns against 5 of 1024:
  // 34.6 / 35.2 on 34816 rows).
  static const int env_r = qs_env("GLOWQ_QSTREAM_R", 0);
  p.r = (env_r == 4 && p.tok <= 4) ? 4 : 2;
  p.slices = (U + 16 * qs_c(p.r) - 1) / (16 * qs_c(p.r));
  if (p.slices > 16) return false;  // (a workgroup's waves)
  // A workgroup is one tile (its slices), or as many tiles as make four waves (the staging counts on 256 threads and
  // more; a workgroup holds at most four tiles).  Small workgroups start and finish independently of each other, which
  // is worth more than the activations they stage redundantly: 8B-shape gate|up at four token rows, 4 / 8 / 16 waves:
  // 17.6 / 20.1 / 20.0 us, o_proj 5.0 / 6.1 / 9.4.
  int waves = p.slices;
  if (env_waves >= 1 && env_waves <= 16) waves = env_waves / p.slices * p.slices;
  if (waves < p.slices) waves = p.slices;
  while (waves < 4) waves += p.slices;
  // each thread stages at most two 16-byte words of a token row (one with eight token rows, or the registers run out)
  const int max_words = p.tok == 8 ? 1 : 2;
  while (waves * kWave * max_words < (K >> 3) && waves + p.slices <= 16 && waves / p.slices < 4) waves += p.slices;
  if (waves > 16 || waves / p.slices > 4) return false;
  if (tiles_per_wg > waves / p.slices) waves = tiles_per_wg * p.slices;
  if (waves > 16 || waves / p.slices > 4) return false;
  p.waves = waves;
  const int threads = waves * kWave, words = K >> 3;
  const int need = (words + threads - 1) / threads;
  p.xw = need <= 1 ? 1 : 2;
  if (need > 2 || (p.tok == 8 && p.xw > 1)) return false;  // (eight token rows: one word each, or the registers run out)
  if (has_r && (rank >> 1) > threads) return false;
  p.lds = qs_lds(p.tok, K, has_r ? rank : 0, waves, p.r).total;
  return p.lds <= 160 * 1024;
}

template <int kR, int kLD, int kTok, int kXW>
hipError_t launch_qs_t(GroupDev& g, const QsPlan& p, hipStream_t stream) {
  auto kern = gemv_qstream_kernel<kR, kLD, kTok, kXW>;
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), p.lds, lds_limit); e != hipSuccess) return e;
  const int tiles_per_wg = p.waves / p.slices;
  int total = 0, grid = 0;
  for (int i = 0; i < g.n_members; ++i) {
    const int tiles = (g.mem[i].N + 4 * kR - 1) / (4 * kR);
    total += tiles;
    g.task_end[i] = total;
    grid += (tiles + tiles_per_wg - 1) / tiles_per_wg;
    g.wg_end[i] = grid;
  }
  // More workgroups than the compute units hold at once: launch as many as they hold and let each walk its share of
  // the list (GLOWQ_QSTREAM_PERSIST=0: one workgroup per entry of the list)
  static const int env_persist = qs_env("GLOWQ_QSTREAM_PERSIST", 1);
  int launch = grid;
  if (env_persist && p.num_cus > 0) {
    static std::atomic<long> seen_key{-1};
    static std::atomic<int> seen_val{0};
    const long key = ((long)p.waves << 32) | (long)p.lds;
    int per_cu = seen_val.load(std::memory_order_acquire);
    if (seen_key.load(std::memory_order_acquire) != key || per_cu <= 0) {
      per_cu = 0;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), p.waves * kWave, p.lds) != hipSuccess || per_cu <= 0)
        per_cu = 0;
      seen_val.store(per_cu, std::memory_order_release);
      seen_key.store(key, std::memory_order_release);
    }
    if (per_cu > 0 && grid > p.num_cus * per_cu) launch = p.num_cus * per_cu;
  }
  hipLaunchKernelGGL(kern, dim3(launch), dim3(p.waves * kWave), p.lds, stream, g, p.slices, tiles_per_wg, grid);
  return hipGetLastError();
}

template <int kLD>
hipError_t launch_qs_x(GroupDev& g, const QsPlan& p, hipStream_t stream) {
#define GLOWQ_CASE(RR, TT, XX) \
  if (p.r == RR && p.tok == TT && p.xw == XX) return launch_qs_t<RR, kLD, TT, XX>(g, p, stream);
  GLOWQ_CASE(4, 2, 1) GLOWQ_CASE(4, 2, 2) GLOWQ_CASE(4, 4, 1) GLOWQ_CASE(4, 4, 2)
  GLOWQ_CASE(2, 2, 1) GLOWQ_CASE(2, 2, 2) GLOWQ_CASE(2, 4, 1) GLOWQ_CASE(2, 4, 2)
#undef GLOWQ_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_qs_l(GroupDev& g, const QsPlan& p, hipStream_t stream) {
  if (g.r == nullptr) return launch_qs_x<0>(g, p, stream);
  return g.rank <= 128 ? launch_qs_x<4>(g, p, stream) : launch_qs_x<8>(g, p, stream);
}

bool aligned_to(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

// 2..4 token rows from the canonical buffers, groups of 128 to 2048 columns (a power of two of 32-column units: the
// caller's layout check), rank a multiple of 8 up to 128 or of 16 up to 256, buffers addressable with 32-bit offsets.
bool qstream_supported(const GroupDev& g) {
  if (g.M < 2 || g.M > 4 || g.group_size < 128 || g.group_size > 2048 || (g.K & 31) != 0 || !aligned_to(g.x, 16)) return false;
  const bool has_r = g.r != nullptr || g.R != nullptr;
  if (has_r) {
    if (g.rank < 8 || g.rank > 256 || (g.rank & 7) != 0 || (g.rank > 128 && (g.rank & 15) != 0)) return false;
    if (g.r != nullptr && !aligned_to(g.r, 4)) return false;
  }
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if (!aligned_to(m.qweight, 16) || (m.ldw & 3) != 0 || !aligned_to(m.qzeros, 4) || !aligned_to(m.scales, 2)) return false;
    if (m.L != nullptr && !aligned_to(m.L, 16)) return false;
    if (m.N >= (1 << 24) || (long)m.ldw * 4 >= (1 << 24) || (long)m.lds * 2 >= (1 << 24) || (long)m.ldz * 4 >= (1 << 24)) return false;
    const long lim = 1L << 31;
    if ((long)m.N * m.ldw * 4 >= lim || (long)m.N * m.lds * 2 >= lim || (long)m.N * m.ldz * 4 >= lim ||
        (has_r && (long)m.N * g.rank * 2 >= lim))
      return false;
  }
  QsPlan p;
  return qs_plan(g.M, g.K, g.rank, has_r, 0, p);
}

hipError_t launch_qstream(GroupDev& g, int num_cus, hipStream_t stream) {
  static const int env_waves = qs_env("GLOWQ_QSTREAM_WAVES", 0);
  QsPlan p;
  if (!qs_plan(g.M, g.K, g.rank, g.r != nullptr, 0, p)) return hipErrorInvalidValue;
  // A launch of few workgroups is over when the compute unit with the most tiles is done: more tiles per workgroup
  // where all workgroups then fit the compute units one each and the most loaded unit has fewer tiles (5120 rows of
  // 5120 columns, 640 tiles on 256 units: two tiles per workgroup leave 64 units with four tiles, three leave every
  // unit with three at most: 9.4 -> 8.3 us at four token rows).
  if (env_waves == 0) {
    auto workgroups = [&](int t) {
      long n = 0;
      for (int i = 0; i < g.n_members; ++i) n += ((g.mem[i].N + 4 * p.r - 1) / (4 * p.r) + t - 1) / t;
      return n;
    };
    const int t0 = p.waves / p.slices;
    const long wgs0 = workgroups(t0);
    if (wgs0 > num_cus && wgs0 <= 2L * num_cus) {
      long best = 2L * t0;
      int pick = t0;
      for (int t = t0 + 1; t <= 4; ++t) {
        QsPlan q;
        if (workgroups(t) <= num_cus && t < best && qs_plan(g.M, g.K, g.rank, g.r != nullptr, t, q)) {
          best = t;
          pick = t;
          break;
        }
      }
      if (pick != t0 && !qs_plan(g.M, g.K, g.rank, g.r != nullptr, pick, p)) return hipErrorInvalidValue;
    }
  }
  p.num_cus = num_cus;
  return launch_qs_l(g, p, stream);
}

}  // namespace glowq
