// Decode GEMV for gfx950: W4A16 linear fused with the group-shared low-rank correction.
//
// One launch covers every member of a group (q|k|v, gate|up, or a solo module).  A wave owns kRows
// output rows and the whole K extent; lane l handles the 16-byte "units" (32 int4 codes) l, l+64,
// ... of each row, so every weight load is a fully coalesced 128-bit load of the canonical
// [N, K/8] int32 layout.  The activations are staged once per workgroup in LDS, already permuted into
// the order the nibble extraction produces, together with the per-unit sums needed to fold the
// zero-point:  sum_k (c - z) s x = s (sum c x - z sum x).
//
// int4 -> fp16 without conversion instructions: a code left in the low mantissa bits of an fp16
// with a zero exponent field is the subnormal c * 2^-24 (c * 2^-20 for the nibble four bits higher),
// exact, and v_dot2_f32_f16 multiplies it by x with fp32 accumulation.  Two accumulators keep the two
// scalings apart; the common 2^24 is applied once per output.
#include <cstdlib>

#include "common.hpp"

namespace glowq {

// Activation staging shared by every wave-dot instantiation.
//   xs  [M][4][U] units of 8 halves: quarter j of unit u holds x[32u + 8j + {0,4,1,5,2,6,3,7}]
//   sig [M][U]    float: 2^-24 * sum of the 32 activations of unit u
//   rs  [M][rank] halves (only when a correction is applied)
// LDS layout of the wave-dot route: x tiles, per-unit sums, then r at a 16-byte aligned offset.
__host__ __device__ inline size_t wave_dot_r_offset(int M, int K) {
  const size_t off = (size_t)M * K * sizeof(half_t) + (size_t)M * (K >> 5) * sizeof(float);
  return (off + 15) & ~(size_t)15;
}

// Total LDS bytes of a workgroup: the above plus M rows of r.
__host__ __device__ inline size_t wave_dot_lds_total(int M, int K, int rank) {
  return (wave_dot_r_offset(M, K) + (size_t)M * rank * sizeof(half_t) + 15) & ~(size_t)15;
}

template <int kM>
__device__ __forceinline__ void stage_activations(const GroupDev& g, int U, h8* xs, float* sig, half_t* rs) {
  const int words = g.K >> 3;  // 8 halves each
  constexpr int kMaxW = 4;     // words of a token row per thread on the short path
  const int rd = g.rank >> 1;
  if (words <= kMaxW * (int)blockDim.x &&
      (g.r == nullptr || ((g.rank & 1) == 0 && rd <= (int)blockDim.x && (reinterpret_cast<uintptr_t>(g.r) & 3u) == 0))) {
    // every request of the staging goes out before anything is used: one memory round trip, not two per token row
    h8 v[kM][kMaxW];
    uint32_t rv[kM];
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      const h8* xrow = reinterpret_cast<const h8*>(g.x + (size_t)m * g.K);
#pragma unroll
      for (int c = 0; c < kMaxW; ++c) {
        const int w = (int)threadIdx.x + c * (int)blockDim.x;
        if (w < words) v[m][c] = xrow[w];
        else v[m][c] = __builtin_nondeterministic_value(v[m][c]);  // never used
      }
      rv[m] = (g.r != nullptr && (int)threadIdx.x < rd) ? reinterpret_cast<const uint32_t*>(g.r + (size_t)m * g.rank)[threadIdx.x] : 0u;
    }
#pragma unroll
    for (int m = 0; m < kM; ++m) {
#pragma unroll
      for (int c = 0; c < kMaxW; ++c) {
        const int w = (int)threadIdx.x + c * (int)blockDim.x;
        if (w < words) {  // words is a multiple of 4: whole quads of threads take this branch
          const h8 q = v[m][c];
          h8 p;
          p[0] = q[0]; p[1] = q[4]; p[2] = q[1]; p[3] = q[5];
          p[4] = q[2]; p[5] = q[6]; p[6] = q[3]; p[7] = q[7];
          const int u = w >> 2, j = w & 3;
          xs[((size_t)m * 4 + j) * U + u] = p;
          float sum = ((float)q[0] + (float)q[1]) + ((float)q[2] + (float)q[3]) +
                      (((float)q[4] + (float)q[5]) + ((float)q[6] + (float)q[7]));
          sum = quad_sum(sum);
          if (j == 0) sig[m * U + u] = sum * 0x1p-24f;
        }
      }
      if (g.r != nullptr && (int)threadIdx.x < rd) reinterpret_cast<uint32_t*>(rs + m * g.rank)[threadIdx.x] = rv[m];
    }
    return;
  }
  for (int m = 0; m < kM; ++m) {
    const h8* xrow = reinterpret_cast<const h8*>(g.x + (size_t)m * g.K);
    for (int w = threadIdx.x; w < words; w += blockDim.x) {
      const h8 v = xrow[w];
      h8 p;
      p[0] = v[0]; p[1] = v[4]; p[2] = v[1]; p[3] = v[5];
      p[4] = v[2]; p[5] = v[6]; p[6] = v[3]; p[7] = v[7];
      const int u = w >> 2, j = w & 3;
      xs[((size_t)m * 4 + j) * U + u] = p;
      float s = ((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3]) +
                (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
      s = quad_sum(s);  // the four quarters of a unit sit in one quad (words is a multiple of 4)
      if (j == 0) sig[m * U + u] = s * 0x1p-24f;
    }
    if (g.r != nullptr) {
      for (int i = threadIdx.x; i < g.rank; i += blockDim.x) rs[m * g.rank + i] = g.r[(size_t)m * g.rank + i];
    }
  }
}

// The same staging for one token row in two halves: the loads go out at the head of the kernel, from pointers that
// arrive in scalar registers, and are written to LDS when the rest of the set-up is done.  Thread t holds words
// t, t + blockDim, ... (at most kXWords) and two halves of r.
constexpr int kXWords = 4;
struct XRegs {
  h8 v[kXWords];
  uint32_t r;
};
__device__ __forceinline__ bool early_staging_fits(int K, int rank, const half_t* r, int threads) {
  return (K >> 3) <= kXWords * threads && (r == nullptr || (rank <= 2 * threads && (reinterpret_cast<uintptr_t>(r) & 3u) == 0));
}
__device__ __forceinline__ void load_activations(const half_t* x, const half_t* r, int K, int rank, int threads, XRegs& xr) {
  const int words = K >> 3;
  const h8* xrow = reinterpret_cast<const h8*>(x);
#pragma unroll
  for (int i = 0; i < kXWords; ++i) xr.v[i] = xrow[min((int)threadIdx.x + i * threads, words - 1)];
  xr.r = 0u;
  if (r != nullptr) xr.r = reinterpret_cast<const uint32_t*>(r)[min((int)threadIdx.x, (rank >> 1) - 1)];
}
__device__ __forceinline__ void store_activations(const half_t* r, int K, int rank, int threads, int U, const XRegs& xr,
                                                  h8* xs, float* sig, half_t* rs) {
  const int words = K >> 3;
#pragma unroll
  for (int i = 0; i < kXWords; ++i) {
    const int w = threadIdx.x + i * threads;
    const h8 v = xr.v[i];
    float s = ((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3]) +
              (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
    s = quad_sum(s);  // threads and words are multiples of 4: a quad lies inside the row or outside as a whole
    if (w < words) {
      h8 p;
      p[0] = v[0]; p[1] = v[4]; p[2] = v[1]; p[3] = v[5];
      p[4] = v[2]; p[5] = v[6]; p[6] = v[3]; p[7] = v[7];
      const int u = w >> 2, j = w & 3;
      xs[(size_t)j * U + u] = p;
      if (j == 0) sig[u] = s * 0x1p-24f;
    }
  }
  if (r != nullptr && (int)threadIdx.x < (rank >> 1)) reinterpret_cast<uint32_t*>(rs)[threadIdx.x] = xr.r;
}

__device__ __forceinline__ void dot_word(uint32_t w, const h8& xq, float& accA, float& accB) {
  // nibbles (0,4) and (2,6) land in mantissa bits 0-3, nibbles (1,5) and (3,7) in bits 4-7.
  const uint32_t hi = w >> 8;
  const h2 c04 = bitcast_u32<h2>(w & 0x000F000Fu);
  const h2 c15 = bitcast_u32<h2>(w & 0x00F000F0u);
  const h2 c26 = bitcast_u32<h2>(hi & 0x000F000Fu);
  const h2 c37 = bitcast_u32<h2>(hi & 0x00F000F0u);
  const h2 x04 = {xq[0], xq[1]};
  const h2 x15 = {xq[2], xq[3]};
  const h2 x26 = {xq[4], xq[5]};
  const h2 x37 = {xq[6], xq[7]};
  accA = __builtin_amdgcn_fdot2(c04, x04, accA, false);
  accB = __builtin_amdgcn_fdot2(c15, x15, accB, false);
  accA = __builtin_amdgcn_fdot2(c26, x26, accA, false);
  accB = __builtin_amdgcn_fdot2(c37, x37, accB, false);
}

// What a wave loads for one row block, all of it issued before anything is used: per row one
// 16-byte unit of 32 int4 codes, the raw scale and zero-point word of the unit's quantisation group,
// and kLW dwords (two halves each) of the row of the left factor L.
// kSide 1: a step holds at most 16 quantisation groups per row (group_size >= 128); then lane 16r + i loads the
// scale and zero-point of group i of row r once per step and the lanes that need it fetch it with ds_bpermute,
// instead of every lane loading its own copy for every row.
// kSide 2 (at most two rows per block, an even number of steps per row block): lane 32r + i loads group i of row r
// of a PAIR of steps with the first step of the pair; the second step issues no scale or zero-point request at all.
// The steps of a pair always sit in the same two prefetch buffers, so every step has a fixed number of loads.
template <int kRows, int kLW, int kSide>
struct Prefetch {
  u32x4 w[kRows];
  half_t sc[kSide ? 1 : kRows];
  uint32_t zw[kSide ? 1 : kRows];
  uint32_t l[kRows][kLW > 0 ? kLW : 1];
};

// Work decomposition.  A row block is kRows consecutive output rows of one member; a wave owns whole
// row blocks, so no partial sums ever cross waves and the only barrier of the kernel is the one after
// the activations are staged.  The K extent is cut into `kit` slices of 2048 columns (64 units, one per
// lane); a step is one slice of one row block and always has the same static shape: kRows coalesced
// 1 KB loads plus the small loads that go with them, all issued one step ahead of their use.
// The correction rides along as a K-extension, y = [deq(W) | L] . [x ; alpha r], the L row being spread
// over the kit steps of its row block (kLW dwords per lane and step).
// Every workgroup serves ONE member for its whole life (the host splits the grid between the members in
// proportion to their row blocks), so the member's pointers and strides are loop invariants held in
// scalar registers and nothing is looked up in memory between two prefetches.
template <int kM, int kRows, int kLW, int kSide>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(((kM >= 2 || kRows >= 4) ? 4 : 6), 8)))
void gemv_wave_dot_kernel(const int32_t* __restrict__ head_qweight, const half_t* __restrict__ head_x,
                          const half_t* __restrict__ head_r, const int head_ldw, const int head_rows,
                          const int head_blocks, const int head_wg_end, const int head_units, const int head_waves,
                          const int head_rank, const GroupDev g, const int kit) {
  // The head_* arguments repeat what a workgroup of the FIRST member needs to request the weights of its first step:
  // plain leading arguments reach the wave in scalar registers, everything inside `g` takes a load from the argument
  // buffer (a memory round trip).  Those workgroups -- all of them for a group of one -- start that much earlier.
  constexpr bool kWide = kSide != 0, kPair = kSide == 2;
  static_assert(!kPair || kRows <= 2, "a pair of steps of one row fills 32 lanes");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int U = g.K >> 5;                                  // 16-byte units per weight row
  const int upg_shift = __builtin_ctz(g.group_size >> 5);  // units per quantisation group = 1 << upg_shift
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + (size_t)kM * g.K * sizeof(half_t));
  half_t* rs = reinterpret_cast<half_t*>(smem + wave_dot_r_offset(kM, g.K));

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  Prefetch<kRows, kLW, kSide> buf0, buf1;
  const bool head = (int)blockIdx.x < head_wg_end;
  if (head) {
    const int n0 = min((int)blockIdx.x * head_waves + wave, head_blocks - 1) * kRows;
    const int u = min(lane, head_units - 1);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int n = min(n0 + r, head_rows - 1);
      buf0.w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(head_qweight + (size_t)n * head_ldw) + u);
    }
  }
  // single token row: the activations (and r) are requested here as well, from leading arguments
  XRegs xr;
  const bool early_x = kM == 1 && early_staging_fits(head_units << 5, head_rank, head_r, head_waves * kWave);
  if (kM == 1 && early_x) load_activations(head_x, head_r, head_units << 5, head_rank, head_waves * kWave, xr);
  const int waves_per_block = blockDim.x >> 6;

  // member of this workgroup: every candidate field comes from a fixed kernel-argument offset and is
  // picked with scalar selects, so the whole lookup costs one round trip to the argument buffer
  MemberDev mem = g.mem[0];
  int wg_begin = 0, wg_stop = g.wg_end[0], total_blocks = g.task_end[0];
#define GLOWQ_PICK(i)                                            \
  if (g.n_members > i && (int)blockIdx.x >= g.wg_end[i - 1]) {  \
    mem = g.mem[i];                                              \
    wg_begin = g.wg_end[i - 1];                                  \
    wg_stop = g.wg_end[i];                                       \
    total_blocks = g.task_end[i] - g.task_end[i - 1];            \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  const int stride = (wg_stop - wg_begin) * waves_per_block;  // waves serving this member
  const int ldw_half = g.rank >> 1;                                // dwords per L row
  const float alpha_scaled = (mem.L != nullptr ? g.alpha : 0.f) * 0x1p-24f;  // accumulators carry 2^-24

  // (row block, slice) of a step; a cursor that ran past the end keeps prefetching the last valid
  // block (valid addresses) and its steps are never computed
  struct Cursor {
    int blk, it;
  };
  const int side_row = min(kPair ? lane >> 5 : lane >> 4, kRows - 1), side_idx = kPair ? lane & 31 : lane & 15;
  const int gps_shift = 6 - upg_shift;  // log2 of the groups per row and step
  // first group of the step (of the pair of steps) whose scales and zero-points the side lanes hold
  auto l_step = [&](int it) { return kPair ? it >> 1 : it; };
  auto side_base = [&](int it) { return kPair ? (it >> 1) << (gps_shift + 1) : it << gps_shift; };
  auto issue = [&](const Cursor& c, Prefetch<kRows, kLW, kSide>& p, const bool weights_requested, const bool with_side) {
    const int n0 = min(c.blk, total_blocks - 1) * kRows;
    const int u = min(lane + c.it * kWave, U - 1);
    const int grp = u >> upg_shift;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int n = min(n0 + r, mem.N - 1);
      if (!weights_requested)
        p.w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(mem.qweight + (size_t)n * mem.ldw) + u);
      if constexpr (!kWide) {
        p.sc[r] = mem.scales[(size_t)n * mem.lds + grp];
        p.zw[r] = (uint32_t)mem.qzeros[(size_t)n * mem.ldz + (grp >> 3)];
      }
      if constexpr (kLW > 0) {
        if (!kPair || with_side) {  // kSide 2: the L row is spread over the first steps of the pairs only
          // a member without L reads r itself (valid memory) and is weighted by zero
          const uint32_t* lrow = mem.L ? reinterpret_cast<const uint32_t*>(mem.L + (size_t)n * g.rank)
                                       : reinterpret_cast<const uint32_t*>(g.r);
#pragma unroll
          for (int j = 0; j < kLW; ++j) p.l[r][j] = lrow[min((l_step(c.it) * kLW + j) * kWave + lane, ldw_half - 1)];
        }
      }
    }
    if constexpr (kWide) {
      if (!kPair || with_side) {  // a constant at every call site
        const int n = min(n0 + side_row, mem.N - 1);
        const int sg = min(side_base(c.it) + side_idx, (U - 1) >> upg_shift);
        p.sc[0] = mem.scales[(size_t)n * mem.lds + sg];
        p.zw[0] = (uint32_t)mem.qzeros[(size_t)n * mem.ldz + (sg >> 3)];
      }
    }
  };
  auto advance = [&](Cursor& c) {
    if (++c.it == kit) {
      c.it = 0;
      c.blk += stride;
    }
  };

  float tot[kRows][kM];
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int m = 0; m < kM; ++m) tot[r][m] = 0.f;

  uint32_t side_held = 0;  // kSide 2: scale and zero-point of this lane's group, packed, kept from the first step of a pair
  auto compute = [&](const Cursor& c, const Prefetch<kRows, kLW, kSide>& p, const bool with_side) {
    const int uraw = lane + c.it * kWave;
    const bool active = uraw < U;
    const int u = active ? uraw : U - 1;
    const int grp = u >> upg_shift;
    float sc[kRows], zp[kRows];
    if constexpr (kWide) {
      const int sg = min(side_base(c.it) + side_idx, (U - 1) >> upg_shift);
      uint32_t packed;
      if (!kPair || with_side) {
        packed = (uint32_t)__builtin_bit_cast(uint16_t, p.sc[0]) | (nibble(p.zw[0], sg & 7) << 16);
        side_held = packed;
      } else {
        packed = side_held;
      }
      const int grel = grp - side_base(c.it);
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const uint32_t sv = (uint32_t)__builtin_amdgcn_ds_bpermute(((kPair ? 32 : 16) * r + grel) << 2, (int)packed);
        sc[r] = active ? (float)__builtin_bit_cast(half_t, (uint16_t)(sv & 0xFFFFu)) : 0.f;
        zp[r] = (float)(sv >> 16);
      }
    } else {
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        sc[r] = active ? (float)p.sc[r] : 0.f;
        zp[r] = (float)nibble(p.zw[r], grp & 7);
      }
    }
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      h8 xq[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) xq[j] = xs[((size_t)m * 4 + j) * U + u];
      const float sg = sig[m * U + u];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        float accA = 0.f, accB = 0.f;
        dot_word(p.w[r].x, xq[0], accA, accB);
        dot_word(p.w[r].y, xq[1], accA, accB);
        dot_word(p.w[r].z, xq[2], accA, accB);
        dot_word(p.w[r].w, xq[3], accA, accB);
        float v = __builtin_fmaf(accB, 0.0625f, accA);
        v = __builtin_fmaf(-zp[r], sg, v);
        tot[r][m] = __builtin_fmaf(sc[r], v, tot[r][m]);
      }
    }
    if (kLW > 0 && (!kPair || with_side)) {
#pragma unroll
      for (int j = 0; j < kLW; ++j) {
        const int idx = (l_step(c.it) * kLW + j) * kWave + lane;
        const float a = idx < ldw_half ? alpha_scaled : 0.f;
        const int ic = min(idx, ldw_half - 1);
#pragma unroll
        for (int m = 0; m < kM; ++m) {
          const h2 rv = reinterpret_cast<const h2*>(rs + m * g.rank)[ic];
#pragma unroll
          for (int r = 0; r < kRows; ++r)
            tot[r][m] = __builtin_fmaf(a, __builtin_amdgcn_fdot2(bitcast_u32<h2>(p.l[r][j]), rv, 0.f, false), tot[r][m]);
        }
      }
    }
    if (c.it == kit - 1) {
      // lane r keeps the total of row r: one store (and one bias load) per token row instead of one per output
      const int n = c.blk * kRows + lane;
      const bool writer = lane < kRows && n < mem.N;
      const float b = (writer && mem.bias) ? (float)mem.bias[n] : 0.f;
#pragma unroll
      for (int m = 0; m < kM; ++m) {
        float mine = 0.f;
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          const float v = wave_sum(tot[r][m]);
          tot[r][m] = 0.f;
          mine = lane == r ? v : mine;
        }
        if (writer) mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(mine, 0x1p24f, b));
      }
    }
  };

  // Software pipeline: the loads of step s+1 are in flight while step s is computed.  The first
  // loads go out before the activations are staged, so the staging hides behind HBM latency.
  Cursor ahead;
  ahead.blk = ((int)blockIdx.x - wg_begin) * waves_per_block + wave;
  ahead.it = 0;
  issue(ahead, buf0, head, true);

  if (kM == 1 && early_x) store_activations(head_r, head_units << 5, head_rank, head_waves * kWave, U, xr, xs, sig, rs);
  else stage_activations<kM>(g, U, xs, sig, rs);
  __syncthreads();

  while (ahead.blk < total_blocks) {
    Cursor cur = ahead;
    advance(ahead);
    issue(ahead, buf1, false, false);
    compute(cur, buf0, true);
    if (ahead.blk >= total_blocks) break;
    cur = ahead;
    advance(ahead);
    issue(ahead, buf0, false, true);
    compute(cur, buf1, false);
  }
}

// Generic route: any K, any alignment, group_size a multiple of 8.  One wave per output row, one
// token row per blockIdx.y; lanes stride over the int32 words of the row.
__global__ __launch_bounds__(256) void gemv_generic_kernel(const GroupDev g) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int total_tasks = g.task_end[g.n_members - 1];
  const int m = blockIdx.y;
  const half_t* x = g.x + (size_t)m * g.K;
  const int words = (g.K + 7) >> 3;
  for (int task = blockIdx.x * waves_per_block + wave; task < total_tasks; task += gridDim.x * waves_per_block) {
    int mi = 0;
    while (mi + 1 < g.n_members && task >= g.task_end[mi]) ++mi;
    const MemberDev& mem = g.mem[mi];
    const int n = task - (mi ? g.task_end[mi - 1] : 0);
    const int32_t* wrow = mem.qweight + (size_t)n * mem.ldw;
    float acc = 0.f;
    for (int w = lane; w < words; w += kWave) {
      const int k0 = w << 3;
      const int grp = k0 / g.group_size;
      const float s = (float)mem.scales[(size_t)n * mem.lds + grp];
      const float z = (float)nibble((uint32_t)mem.qzeros[(size_t)n * mem.ldz + (grp >> 3)], grp & 7);
      const uint32_t pw = (uint32_t)wrow[w];
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k = k0 + i;
        const float xv = (k < g.K) ? (float)x[k] : 0.f;
        part = __builtin_fmaf((float)nibble(pw, i) - z, xv, part);
      }
      acc = __builtin_fmaf(s, part, acc);
    }
    if (mem.L != nullptr && g.r != nullptr) {
      float corr = 0.f;
      for (int j = lane; j < g.rank; j += kWave)
        corr = __builtin_fmaf((float)mem.L[(size_t)n * g.rank + j], (float)g.r[(size_t)m * g.rank + j], corr);
      acc = __builtin_fmaf(g.alpha, corr, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      const float b = mem.bias ? (float)mem.bias[n] : 0.f;
      mem.y[(size_t)m * mem.ldy + n] = (half_t)(acc + b);
    }
  }
}

// ---- host launchers ---------------------------------------------------------------------
size_t wave_dot_lds_bytes(int M, int K, int rank, bool has_r) {
  return wave_dot_lds_total(M, K, has_r ? rank : 0);
}

static int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

// Launch tuning knobs (rows per row block, waves per workgroup, cap on workgroups per CU); the
// environment overrides exist for tuning runs and are read once.
struct WaveDotTuning {
  int rows, waves, max_wg_per_cu;
};
static const WaveDotTuning& tuning_override() {
  static const WaveDotTuning t = {env_int("GLOWQ_GEMV_ROWS", 0), env_int("GLOWQ_GEMV_WAVES", 0),
                                  env_int("GLOWQ_GEMV_WG_PER_CU", 0)};
  return t;
}

template <int kM, int kRows, int kLW, int kSide>
static hipError_t launch_wave_dot_t(const GroupDev& g, int kit, int waves, int max_wg_per_cu, int num_cus, size_t lds,
                                    hipStream_t stream) {
  auto kern = gemv_wave_dot_kernel<kM, kRows, kLW, kSide>;
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
  // resident workgroups per CU for a block size and LDS footprint; each host thread remembers its last answers
  auto occupancy = [&](int threads, int& occ) -> hipError_t {
    static thread_local int last_threads[3] = {0, 0, 0}, last_occ[3] = {0, 0, 0};
    static thread_local size_t last_lds[3] = {0, 0, 0};
    const int slot = threads == 8 * kWave ? 0 : (threads == 7 * kWave ? 1 : 2);
    if (last_occ[slot] == 0 || last_threads[slot] != threads || last_lds[slot] != lds) {
      int o = 0;
      hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, reinterpret_cast<const void*>(kern), threads, lds);
      if (e != hipSuccess) return e;
      last_threads[slot] = threads;
      last_lds[slot] = lds;
      last_occ[slot] = o < 1 ? 1 : o;
    }
    occ = last_occ[slot];
    if (max_wg_per_cu > 0 && occ > max_wg_per_cu) occ = max_wg_per_cu;
    return hipSuccess;
  };
  // Split the grid between the members in proportion to their row blocks; when everything does not
  // fit on the chip at once the waves become persistent and walk an equal number of row blocks.
  static const int persist = env_int("GLOWQ_GEMV_PERSIST", 1);
  struct Plan {
    int grid, rounds, wg_end[GLOWQ_MAX_MEMBERS];
    double cost;  // time of the most loaded CU over the mean, times the same for the most loaded wave
  };
  auto plan = [&](int w, int occ) {
    Plan p;
    const int resident = num_cus * occ;
    int wgs_needed = 0;
    for (int i = 0; i < g.n_members; ++i) {
      const int blocks = g.task_end[i] - (i ? g.task_end[i - 1] : 0);
      wgs_needed += (blocks + w - 1) / w;
    }
    p.rounds = (persist != 0 && wgs_needed > resident) ? (wgs_needed + resident - 1) / resident : 1;
    p.grid = 0;
    double wave_imbalance = 1.0;
    for (int i = 0; i < g.n_members; ++i) {
      const int blocks = g.task_end[i] - (i ? g.task_end[i - 1] : 0);
      int wg_i = ((blocks + w - 1) / w + p.rounds - 1) / p.rounds;
      if (wg_i < 1) wg_i = 1;
      p.grid += wg_i;
      p.wg_end[i] = p.grid;
      const long slots = (long)wg_i * w;
      const double imb = (double)((blocks + slots - 1) / slots * slots) / (double)blocks;
      wave_imbalance = imb > wave_imbalance ? imb : wave_imbalance;
    }
    const int per_cu = (p.grid + num_cus - 1) / num_cus;
    p.cost = wave_imbalance * (double)per_cu * num_cus / (double)p.grid;
    return p;
  };
  int occ = 1;
  if (hipError_t e = occupancy(waves * kWave, occ); e != hipSuccess) return e;
  Plan chosen = plan(waves, occ);
  // A long single-row group (persistent waves): 7 waves per workgroup where that spreads the workgroups evenly over
  // the CUs and the row blocks evenly over the waves and 8 do not (28672 rows: 512 workgroups of 7 waves, two on every
  // CU, against 448 of 8, two on three quarters of the CUs: 14.5 against 15.1 us).
  if (kM == 1 && waves == 8 && chosen.rounds > 1 && tuning_override().waves == 0) {
    int occ7 = 1;
    if (hipError_t e = occupancy(7 * kWave, occ7); e != hipSuccess) return e;
    const Plan alt = plan(7, occ7);
    if (alt.rounds > 1 && alt.cost < 0.97 * chosen.cost) {
      chosen = alt;
      waves = 7;
    }
  }
  // A group that fits the chip in one go but leaves its workgroups unevenly spread over the CUs (q|k|v of an 8B-shape
  // layer: 384 workgroups of 8 waves on 256 CUs): 4 waves per workgroup where that evens them out (768: three per CU,
  // 6.4 -> 5.9 us).  Evenly spread groups are not touched: o_proj and down_proj lose with 4 waves.
  if (kM == 1 && waves == 8 && chosen.rounds == 1 && tuning_override().waves == 0) {
    int occ4 = 1;
    if (hipError_t e = occupancy(4 * kWave, occ4); e != hipSuccess) return e;
    const Plan alt = plan(4, occ4);
    if (alt.rounds == 1 && alt.cost < 0.9 * chosen.cost) {
      chosen = alt;
      waves = 4;
    }
  }
  const int threads = waves * kWave;
  GroupDev gl = g;
  const int grid = chosen.grid;
  for (int i = 0; i < g.n_members; ++i) gl.wg_end[i] = chosen.wg_end[i];
  hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, stream, gl.mem[0].qweight, gl.x, gl.r, gl.mem[0].ldw, gl.mem[0].N,
                     gl.task_end[0], gl.wg_end[0], gl.K >> 5, waves, gl.r ? gl.rank : 0, gl, kit);
  return hipGetLastError();
}

// The wave-dot route covers K up to 16 slices of 2048 columns and ranks up to 2 dwords per lane
// and slice wave.
bool wave_dot_supported(int M, int K, int rank, bool has_r) {
  const int kit = (K / 32 + kWave - 1) / kWave;
  if (M < 1 || M > 4 || kit > 16) return false;
  if (has_r && (rank & 1)) return false;
  if (has_r && rank > 2 * 128 * kit) return false;
  return wave_dot_lds_bytes(M, K, rank, has_r) <= 160 * 1024;
}

int wave_dot_rows(long total_rows) {
  const int o = tuning_override().rows;
  if (o == 1 || o == 2 || o == 4) return o;
  return total_rows >= 8192 ? 4 : 2;
}
// Single-row decode: two rows per row block throughout (four measured 2 % slower on the long groups once the first
// request of a wave no longer waits for the argument buffer).
int wave_dot_rows_single(long total_rows) {
  const int o = tuning_override().rows;
  if (o == 1 || o == 2 || o == 4) return o;
  (void)total_rows;
  return 2;
}

hipError_t launch_wave_dot(GroupDev& g, int rows_per_block, int num_cus, hipStream_t stream) {
  // register budget: rows x tokens held to 4 accumulators per lane
  while (rows_per_block * g.M > 4) rows_per_block >>= 1;
  int total = 0;
  for (int i = 0; i < g.n_members; ++i) {
    total += (g.mem[i].N + rows_per_block - 1) / rows_per_block;
    g.task_end[i] = total;
  }
  const int kit = (g.K / 32 + kWave - 1) / kWave;
  const bool has_r = g.r != nullptr;
  int lw = has_r ? (g.rank + 128 * kit - 1) / (128 * kit) : 0;
  const size_t lds = wave_dot_lds_bytes(g.M, g.K, g.rank, has_r);
  int waves = tuning_override().waves;
  if (waves < 1 || waves > 16) waves = 8;
  const int max_wg = tuning_override().max_wg_per_cu;
  // the shared scale / zero-point loads pay for single-row decode; the multi-row instantiations keep per-lane loads
  const bool wide = g.M == 1 && g.group_size >= 128;
  static const int env_pair = env_int("GLOWQ_GEMV_PAIR", 1);
  // in pairs the L row rides on every other step: twice the dwords per lane there
  const int lw_pair = has_r ? (g.rank + 64 * kit - 1) / (64 * kit) : 0;
  const bool pair = wide && rows_per_block <= 2 && (kit & 1) == 0 && lw_pair <= 2 && env_pair != 0;
  if (pair) lw = lw_pair;
#define GLOWQ_CASE(MM, RR, LL)                                                                                   \
  if (g.M == MM && rows_per_block == RR && lw == LL) {                                                           \
    if (MM == 1 && pair) return launch_wave_dot_t<MM, RR, LL, (MM == 1 && RR <= 2) ? 2 : 0>(g, kit, waves, max_wg, num_cus, lds, stream); \
    if (MM == 1 && wide) return launch_wave_dot_t<MM, RR, LL, (MM == 1) ? 1 : 0>(g, kit, waves, max_wg, num_cus, lds, stream);           \
    return launch_wave_dot_t<MM, RR, LL, 0>(g, kit, waves, max_wg, num_cus, lds, stream);                         \
  }
#define GLOWQ_CASES(MM, RR) GLOWQ_CASE(MM, RR, 0) GLOWQ_CASE(MM, RR, 1) GLOWQ_CASE(MM, RR, 2)
  GLOWQ_CASES(1, 1) GLOWQ_CASES(1, 2) GLOWQ_CASES(1, 4)
  GLOWQ_CASES(2, 1) GLOWQ_CASES(2, 2)
  GLOWQ_CASES(3, 1)
  GLOWQ_CASES(4, 1)
#undef GLOWQ_CASES
#undef GLOWQ_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_generic(GroupDev& g, int num_cus, hipStream_t stream) {
  int total = 0;
  for (int i = 0; i < g.n_members; ++i) {
    total += g.mem[i].N;
    g.task_end[i] = total;
  }
  int grid = (total + 3) / 4;
  const int cap = num_cus * 8;
  if (grid > cap) grid = cap;
  if (grid < 1) grid = 1;
  hipLaunchKernelGGL(gemv_generic_kernel, dim3(grid, g.M), dim3(256), 0, stream, g);
  return hipGetLastError();
}

}  // namespace glowq
