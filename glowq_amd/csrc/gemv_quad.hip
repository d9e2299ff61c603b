// Decode GEMV for 1..16 token rows on the 4x4x4 matrix cores of gfx950.
//
// v_mfma_f32_4x4x4_16B_f16 multiplies sixteen independent 4x4x4 blocks: lanes 4b..4b+3 form block b, lane
// 4b+q supplies four k values of row q of A and of column q of B, and receives column q of the 4x4 result.
// Here row q of A is token row q of the activations and column q of B is output row n0+q of the weights, so
// ONE instruction pair per 8 codes serves four token rows at the price of one, and four of them sixteen.
//
// The codes are not converted: masked in place they are fp16 subnormals (c * 2^-24 in mantissa bits 0-3,
// c * 2^-20 in bits 4-7), which the matrix core multiplies exactly.  Two accumulators keep the two scalings
// apart; the zero-point is folded through per-unit activation sums, sum (c - z) s x = s (sum c x - z sum x).
//
// Work decomposition: a row block is 4 consecutive output rows of one member; a step is 2048 columns of a
// row block.  Memory is read in the order it lies: in load c lane 16r + i reads unit 16c + i of row n0 + r
// (16 consecutive lanes = 256 contiguous bytes), and the same lanes fetch the scale and zero-point of the
// groups of that step, once.  The matrix core wants block b = unit, column q = row, i.e. lane 4b + q: the
// 4 x 16 -> 16 x 4 lane transposition is done with ds_bpermute on the way into the B operand.  A wave owns
// whole row blocks (or a K-slice of one, see `slices`).  The correction rides along as a K-extension with
// the rows of L as fp16 B operands.
#include <cstdlib>

#include "common.hpp"

namespace glowq {

namespace {

constexpr int kQuadRows = 4;

struct QuadLds {
  int tokens;      // token rows staged (M rounded up to 1, 2 or a multiple of 4)
  int tok4;        // tokens rounded up to a multiple of 4 (row count of sig and rs)
  int x_stride;    // h8 per token row of xs: 4 U + 1 (the odd stride spreads the four tokens of a quad over banks)
  int r_stride;    // halves per token row of rs: rank + 8
  size_t sig_off, r_off, total;
};

__host__ __device__ inline QuadLds quad_lds(int tokens, int K, int rank) {
  QuadLds l;
  const int U = K >> 5;
  l.tokens = tokens;
  l.tok4 = (tokens + 3) & ~3;
  l.x_stride = 4 * U + 1;
  l.r_stride = rank + 8;
  l.sig_off = (size_t)tokens * l.x_stride * 16;
  l.r_off = l.sig_off + (size_t)U * l.tok4 * sizeof(float);
  l.total = l.r_off + (rank > 0 ? (size_t)l.tok4 * l.r_stride * sizeof(half_t) : 0);
  return l;
}

// xs  [tokens][4 U + 1] of 8 halves: word t of unit u of token m at m * x_stride + t * U + u, holding
//     x[32u + 8t + {0,4,2,6, 1,5,3,7}] (the order the two masked operands of a code word come out in)
// sig [U][tok4] floats: 2^-24 * sum of the 32 activations of unit u, per token
// rs  [tok4][rank + 8] halves
// Token rows past M repeat row M-1: their results are computed and never stored.
template <int kM>
__device__ __forceinline__ void stage_quad(const GroupDev& g, const QuadLds& l, h8* xs, float* sig, half_t* rs) {
  const int words = g.K >> 3;
  const int U = g.K >> 5;
  if constexpr (kM <= 4) {
    // Up to four token rows: every request of the staging goes out before anything is used -- one memory round trip
    // instead of two per token row (x, then r), which is most of what a short launch costs.
    constexpr int kMaxW = 4;                 // 16-byte words of a token row per thread
    constexpr int kTok4 = (kM + 3) & ~3;
    const int rd = g.rank >> 1;              // dwords of a row of r
    if (words <= kMaxW * (int)blockDim.x && (g.r == nullptr || rd <= (int)blockDim.x)) {
      h8 v[kM][kMaxW];
      uint32_t rv[kTok4];
#pragma unroll
      for (int m = 0; m < kM; ++m) {
        const h8* xrow = reinterpret_cast<const h8*>(g.x + (size_t)min(m, g.M - 1) * g.K);
#pragma unroll
        for (int c = 0; c < kMaxW; ++c) {
          const int w = (int)threadIdx.x + c * (int)blockDim.x;
          if (w < words) v[m][c] = xrow[w];
          else v[m][c] = __builtin_nondeterministic_value(v[m][c]);  // never used
        }
      }
#pragma unroll
      for (int m = 0; m < kTok4; ++m)
        rv[m] = (g.r != nullptr && (int)threadIdx.x < rd)
                    ? reinterpret_cast<const uint32_t*>(g.r + (size_t)min(m, g.M - 1) * g.rank)[threadIdx.x] : 0u;
#pragma unroll
      for (int m = 0; m < kM; ++m) {
#pragma unroll
        for (int c = 0; c < kMaxW; ++c) {
          const int w = (int)threadIdx.x + c * (int)blockDim.x;
          if (w < words) {  // the four words of a unit sit in one quad of threads: whole quads take this branch
            const h8 q = v[m][c];
            h8 p;
            p[0] = q[0]; p[1] = q[4]; p[2] = q[2]; p[3] = q[6];
            p[4] = q[1]; p[5] = q[5]; p[6] = q[3]; p[7] = q[7];
            const int u = w >> 2, t = w & 3;
            xs[(size_t)m * l.x_stride + t * U + u] = p;
            float sum = ((float)q[0] + (float)q[1]) + ((float)q[2] + (float)q[3]) +
                        (((float)q[4] + (float)q[5]) + ((float)q[6] + (float)q[7]));
            sum = quad_sum(sum);
            if (t == 0) sig[u * l.tok4 + m] = sum * 0x1p-24f;
          }
        }
      }
      for (int m = kM; m < kTok4; ++m)
        for (int u = threadIdx.x; u < U; u += blockDim.x) sig[u * l.tok4 + m] = 0.f;
      if (g.r != nullptr && (int)threadIdx.x < rd) {
#pragma unroll
        for (int m = 0; m < kTok4; ++m) reinterpret_cast<uint32_t*>(rs + m * l.r_stride)[threadIdx.x] = rv[m];
      }
      return;
    }
  }
#pragma unroll 1
  for (int m = 0; m < l.tok4; ++m) {
    const int src = min(m, g.M - 1);
    if (m < kM) {
      const h8* xrow = reinterpret_cast<const h8*>(g.x + (size_t)src * g.K);
      for (int w = threadIdx.x; w < words; w += blockDim.x) {
        const h8 v = xrow[w];
        h8 p;
        p[0] = v[0]; p[1] = v[4]; p[2] = v[2]; p[3] = v[6];
        p[4] = v[1]; p[5] = v[5]; p[6] = v[3]; p[7] = v[7];
        const int u = w >> 2, t = w & 3;
        xs[(size_t)m * l.x_stride + t * U + u] = p;
        float s = ((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3]) +
                  (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
        s = quad_sum(s);  // the four words of a unit sit in one quad of threads
        if (t == 0) sig[u * l.tok4 + m] = s * 0x1p-24f;
      }
    } else {
      for (int u = threadIdx.x; u < U; u += blockDim.x) sig[u * l.tok4 + m] = 0.f;
    }
    if (g.r != nullptr)
      for (int i = threadIdx.x; i < g.rank; i += blockDim.x) rs[m * l.r_stride + i] = g.r[(size_t)src * g.rank + i];
  }
}

// kWide: a step holds at most 16 quantisation groups per row (group_size >= 128), so one scale and one
// zero-point load per lane and step cover them; otherwise every 16-byte unit brings its own.
template <int kLW, bool kWide>
struct QuadPrefetch {
  u32x4 w[4];
  half_t sc[kWide ? 1 : 4];
  uint32_t zw[kWide ? 1 : 4];
  uint32_t l[kLW > 0 ? kLW : 1];
};

__device__ __forceinline__ uint32_t lane_fetch(int src_lane_bytes, uint32_t v) {
  return (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane_bytes, (int)v);
}

// sum over the 16 lanes that share lane % 4; every lane gets the total of its class
__device__ __forceinline__ float quad_class_sum(float v, int lane) {
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true);  // row_ror:4
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true);  // row_ror:8
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, v));
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, v));
  v += __builtin_bit_cast(float, t);
  return v;
}

}  // namespace

// kM: staged token rows (1, 2, 4, 8, 16); kLW: dwords of an L row per lane and step (0, 2 or 4).
// `slices` waves of a workgroup share one row block, each taking a contiguous range of its `kit` steps; their
// partial sums meet in LDS (one barrier per row block).  With slices == 1 a wave owns whole row blocks and the
// only barrier is the one after staging.
template <int kM, int kLW, bool kWide>
__global__ __launch_bounds__(kM > 8 ? 512 : 1024) __attribute__((amdgpu_waves_per_eu((kM > 8 ? 2 : 4), 8)))
void gemv_quad_kernel(const GroupDev g, const int kit, const int slices) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int kSets = (kM + 3) / 4;
  constexpr int kLast = kM - 4 * (kSets - 1);  // token rows of the last set that are worth finishing
  constexpr int kTok4 = 4 * kSets;
  const int U = g.K >> 5;
  const int upg_shift = __builtin_ctz(g.group_size >> 5);
  const QuadLds lay = quad_lds(kM, g.K, g.r ? g.rank : 0);
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + lay.sig_off);
  half_t* rs = reinterpret_cast<half_t*>(smem + lay.r_off);
  float* part = reinterpret_cast<float*>(smem + lay.total);  // [2][waves][kTok4][4 rows], only with slices > 1

  const int lane = threadIdx.x & (kWave - 1);
  const int qb = lane >> 2, qj = lane & 3;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_per_block = blockDim.x >> 6;
  const int blocks_per_wg = waves_per_block / slices;
  const int local_blk = wave / slices, slice = wave - local_blk * slices;
  const int it_begin = (slice * kit) / slices, it_end = ((slice + 1) * kit) / slices;

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
  const int stride = (wg_stop - wg_begin) * blocks_per_wg;
  const int l_chunks = (g.rank >> 1) / (kLW > 0 ? kLW : 1);  // chunks of kLW dwords in an L row
  const bool has_l = kLW > 0 && mem.L != nullptr;
  const float alpha_scaled = (has_l ? g.alpha : 0.f) * 0x1p-24f;  // the accumulators carry 2^-24
  // every member's buffers stay below 2 GiB (checked on the host): uniform base + 32-bit byte offset
  const char* wbase = reinterpret_cast<const char*>(mem.qweight);
  const char* sbase = reinterpret_cast<const char*>(mem.scales);
  const char* zbase = reinterpret_cast<const char*>(mem.qzeros);
  const char* lbase = reinterpret_cast<const char*>(has_l ? mem.L : g.x);  // without L: valid memory, zeroed later
  const uint32_t l_row_bytes = has_l ? (uint32_t)g.rank * 2u : 0u;

  struct Cursor {
    int blk, it;
  };
  const int lr = lane >> 4, lu = lane & 15;  // row and unit-in-load this lane reads from memory
  const int fetch_w = (16 * qj + qb) << 2;    // byte address of the lane that read (row qj, unit qb)
  const int gps_shift = 6 - upg_shift;        // log2 of the groups per row and step
  auto issue = [&](const Cursor& c, QuadPrefetch<kLW, kWide>& p) {
    // A cursor past the end still issues its loads (the pipeline has one static shape), but every lane then
    // reads the first 16 bytes of x: one cached request per load instead of a second pass over a row block.
    const bool valid = c.blk < total_blocks;
    const uint32_t n = (uint32_t)min(c.blk * kQuadRows + lr, mem.N - 1);
    const uint32_t w_row = valid ? n * (uint32_t)mem.ldw * 4u : 0u, s_row = valid ? n * (uint32_t)mem.lds * 2u : 0u,
                   z_row = valid ? n * (uint32_t)mem.ldz * 4u : 0u;
    const char* wb = valid ? wbase : reinterpret_cast<const char*>(g.x);
    const char* sb = valid ? sbase : reinterpret_cast<const char*>(g.x);
    const char* zb = valid ? zbase : reinterpret_cast<const char*>(g.x);
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const uint32_t u = valid ? (uint32_t)min(c.it * kWave + cc * 16 + lu, U - 1) : 0u;
      p.w[cc] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wb + (w_row + u * 16u)));
      if constexpr (!kWide) {
        const uint32_t grp = u >> upg_shift;
        p.sc[cc] = *reinterpret_cast<const half_t*>(sb + (s_row + grp * 2u));
        p.zw[cc] = *reinterpret_cast<const uint32_t*>(zb + (z_row + (grp >> 3) * 4u));
      }
    }
    if constexpr (kWide) {
      const uint32_t grp = valid ? (uint32_t)min((c.it << gps_shift) + lu, (U - 1) >> upg_shift) : 0u;
      p.sc[0] = *reinterpret_cast<const half_t*>(sb + (s_row + grp * 2u));
      p.zw[0] = *reinterpret_cast<const uint32_t*>(zb + (z_row + (grp >> 3) * 4u));
    }
    if constexpr (kLW > 0) {
      const uint32_t nq = (uint32_t)min(c.blk * kQuadRows + qj, mem.N - 1);
      const uint32_t q = valid ? (uint32_t)min(c.it * 16 + qb, l_chunks - 1) : 0u;
      const char* lp = (valid ? lbase : reinterpret_cast<const char*>(g.x)) + ((valid ? nq * l_row_bytes : 0u) + q * (4u * kLW));
      if constexpr (kLW == 2) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(lp);
        p.l[0] = v.x; p.l[1] = v.y;
      } else {
        const u32x4 v = *reinterpret_cast<const u32x4*>(lp);
        p.l[0] = v.x; p.l[1] = v.y; p.l[2] = v.z; p.l[3] = v.w;
      }
    }
  };
  auto advance = [&](Cursor& c) {
    if (++c.it == it_end) {
      c.it = it_begin;
      c.blk += stride;
    }
  };

  f4 tot[kSets], accL[kSets];
#pragma unroll
  for (int s = 0; s < kSets; ++s) {
    tot[s] = f4{0.f, 0.f, 0.f, 0.f};
    accL[s] = f4{0.f, 0.f, 0.f, 0.f};
  }
  int parity = 0;

  auto compute = [&](const Cursor& c, const QuadPrefetch<kLW, kWide>& p) {
    // scale bits and zero-point of the group(s) this lane loaded, packed for the lane exchange
    uint32_t side[kWide ? 1 : 4];
    if constexpr (kWide) {
      const int grp = min((c.it << gps_shift) + lu, (U - 1) >> upg_shift);
      side[0] = (uint32_t)__builtin_bit_cast(uint16_t, p.sc[0]) | (nibble(p.zw[0], grp & 7) << 16);
    } else {
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
        const int grp = min(c.it * kWave + cc * 16 + lu, U - 1) >> upg_shift;
        side[cc] = (uint32_t)__builtin_bit_cast(uint16_t, p.sc[cc]) | (nibble(p.zw[cc], grp & 7) << 16);
      }
    }
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int uraw = c.it * kWave + cc * 16 + qb;
      const bool active = uraw < U;
      const int u = active ? uraw : U - 1;
      uint32_t sv;
      if constexpr (kWide) {
        const int grel = (u >> upg_shift) - (c.it << gps_shift);  // group of this unit within the step
        sv = lane_fetch((16 * qj + grel) << 2, side[0]);
      } else {
        sv = lane_fetch(fetch_w, side[cc]);
      }
      const float sc = active ? (float)__builtin_bit_cast(half_t, (uint16_t)(sv & 0xFFFFu)) : 0.f;
      const float zp = (float)(sv >> 16);
      h4 b_lo[4], b_hi[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t w = lane_fetch(fetch_w, p.w[cc][t]);
        const uint32_t hi = w >> 8;
        b_lo[t] = __builtin_bit_cast(h4, u32x2{w & 0x000F000Fu, hi & 0x000F000Fu});  // codes 0,4,2,6 * 2^-24
        b_hi[t] = __builtin_bit_cast(h4, u32x2{w & 0x00F000F0u, hi & 0x00F000F0u});  // codes 1,5,3,7 * 2^-20
      }
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        const int tok = (kM >= 4) ? 4 * s + qj : min(qj, kM - 1);
        const h8* xt = xs + (size_t)tok * lay.x_stride + u;
        f4 accA = {0.f, 0.f, 0.f, 0.f}, accB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const h8 xv = xt[t * U];
          const h4 a_lo = {xv[0], xv[1], xv[2], xv[3]};
          const h4 a_hi = {xv[4], xv[5], xv[6], xv[7]};
          accA = __builtin_amdgcn_mfma_f32_4x4x4f16(a_lo, b_lo[t], accA, 0, 0, 0);
          accB = __builtin_amdgcn_mfma_f32_4x4x4f16(a_hi, b_hi[t], accB, 0, 0, 0);
        }
        const f4 sg = *reinterpret_cast<const f4*>(sig + u * lay.tok4 + 4 * s);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (s == kSets - 1 && i >= kLast) break;
          float v = __builtin_fmaf(accB[i], 0.0625f, accA[i]);
          v = __builtin_fmaf(-zp, sg[i], v);
          tot[s][i] = __builtin_fmaf(sc, v, tot[s][i]);
        }
      }
    }
    if constexpr (kLW > 0) {
      const int qraw = c.it * 16 + qb;
      const bool live = has_l && qraw < l_chunks;
      const int q = min(qraw, l_chunks - 1);
      uint32_t ld[kLW];
#pragma unroll
      for (int j = 0; j < kLW; ++j) ld[j] = live ? p.l[j] : 0u;
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        const int tok = (kM >= 4) ? 4 * s + qj : min(qj, kM - 1);
        const half_t* rt = rs + tok * lay.r_stride + q * (2 * kLW);
#pragma unroll
        for (int j = 0; j < kLW; j += 2) {
          const h4 a = *reinterpret_cast<const h4*>(rt + 2 * j);
          accL[s] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, __builtin_bit_cast(h4, u32x2{ld[j], ld[j + 1]}), accL[s], 0, 0, 0);
        }
      }
    }
    if (c.it == it_end - 1) {
      // the row block is finished for this wave: reduce over the 16 lanes of each row, then either store
      // (a wave that owns the whole K extent) or leave the partial sums for the first slice to add up
      const int n = c.blk * kQuadRows + qj;
      const bool writer = qb == 0 && c.blk < total_blocks && n < mem.N;
      const float bias = (writer && mem.bias) ? (float)mem.bias[n] : 0.f;
      float* mine = part + ((size_t)(parity * waves_per_block + wave) * kTok4) * 4;
      const float* first = part + ((size_t)(parity * waves_per_block + local_blk * slices) * kTok4) * 4;
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (s == kSets - 1 && i >= kLast) break;
          float v = tot[s][i];
          if constexpr (kLW > 0) v = __builtin_fmaf(alpha_scaled, accL[s][i], v);
          v = quad_class_sum(v, lane);
          const int m = 4 * s + i;
          if (slices > 1) {
            if (qb == 0) mine[m * 4 + qj] = v;
          } else if (writer && m < g.M) {
            mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(v, 0x1p24f, bias));
          }
        }
        tot[s] = f4{0.f, 0.f, 0.f, 0.f};
        accL[s] = f4{0.f, 0.f, 0.f, 0.f};
      }
      if (slices > 1) {
        __syncthreads();  // every wave of the workgroup finishes a row block the same number of times
        parity ^= 1;
        if (slice == 0) {
#pragma unroll
          for (int s = 0; s < kSets; ++s) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (s == kSets - 1 && i >= kLast) break;
              const int m = 4 * s + i;
              float v = 0.f;
              for (int o = 0; o < slices; ++o) v += first[((size_t)o * kTok4 + m) * 4 + qj];
              if (writer && m < g.M) mem.y[(size_t)m * mem.ldy + n] = (half_t)(__builtin_fmaf(v, 0x1p24f, bias));
            }
          }
        }
      }
    }
  };

  // Two-deep software pipeline; the first loads go out before the activations are staged.  All waves of a
  // workgroup walk the same number of row blocks (a wave past the end recomputes the last block and stores
  // nothing), which keeps the barriers of the sliced mode matched.
  const int first_blk = ((int)blockIdx.x - wg_begin) * blocks_per_wg;
  const int rounds = first_blk < total_blocks ? (total_blocks - 1 - first_blk) / stride + 1 : 0;
  int steps = rounds * (it_end - it_begin);
  Cursor ahead;
  ahead.blk = first_blk + local_blk;
  ahead.it = it_begin;
  QuadPrefetch<kLW, kWide> buf0, buf1;
  issue(ahead, buf0);

  stage_quad<kM>(g, lay, xs, sig, rs);
  __syncthreads();

  while (steps > 0) {
    Cursor cur = ahead;
    advance(ahead);
    issue(ahead, buf1);
    compute(cur, buf0);
    if (--steps == 0) break;
    cur = ahead;
    advance(ahead);
    issue(ahead, buf0);
    compute(cur, buf1);
    --steps;
  }
}

// ---- host side ------------------------------------------------------------------------------
static int quad_tokens(int M) { return M <= 2 ? M : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)); }

static int quad_env(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

// dwords of an L row per lane and step: 16 lanes x kit steps cover the rank / 2 dwords of a row
static int quad_lw(int rank, int kit) {
  const int per_lane = (rank / 2 + 16 * kit - 1) / (16 * kit);
  return per_lane <= 2 ? 2 : 4;
}

bool quad_supported(int M, int K, int rank, bool has_r) {
  const int kit = (K / 32 + kWave - 1) / kWave;
  if (M < 1 || M > 16 || kit > 16) return false;
  if (has_r && ((rank & 7) != 0 || rank / 2 > 4 * 16 * kit || rank > K)) return false;
  // room for the slice partial sums: 2 x 16 waves x 16 tokens x 4 rows floats
  return quad_lds(quad_tokens(M), K, has_r ? rank : 0).total + 8192 <= 160 * 1024;
}

template <int kM, int kLW, bool kWide>
static hipError_t launch_quad_t(const GroupDev& g, int kit, int num_cus, size_t lds_base, hipStream_t stream) {
  auto kern = gemv_quad_kernel<kM, kLW, kWide>;
  // 16 waves per CU (8 for the widest token count), in as many workgroups as the LDS footprint allows
  static const int waves_env = quad_env("GLOWQ_QUAD_WAVES", 0);
  static const int wg_env = quad_env("GLOWQ_QUAD_WG_PER_CU", 0);
  static const int slices_env = quad_env("GLOWQ_QUAD_SLICES", 0);
  constexpr int kTok4 = 4 * ((kM + 3) / 4);
  const int cu_waves = kM > 8 ? 8 : 16;
  const size_t part_max = (size_t)2 * 16 * kTok4 * 4 * sizeof(float);
  int wg_per_cu = (int)((160 * 1024) / (lds_base + part_max));
  if (wg_per_cu < 1) wg_per_cu = 1;
  if (wg_per_cu > 2) wg_per_cu = 2;
  if (wg_env >= 1) wg_per_cu = wg_env;
  int waves = cu_waves / wg_per_cu;
  if (waves_env >= 1 && waves_env <= 16) waves = waves_env;
  // slices: when there are fewer row blocks than resident waves, several waves share a row block along K
  const int total_blocks = g.task_end[g.n_members - 1];
  int slices = 1;
  while (slices * 2 <= kit && slices * 2 <= waves && (long)total_blocks * slices * 2 <= (long)num_cus * cu_waves) slices *= 2;
  if (slices_env >= 1 && slices_env <= waves && waves % slices_env == 0 && slices_env <= kit) slices = slices_env;
  const int blocks_per_wg = waves / slices;
  const size_t lds = lds_base + (slices > 1 ? (size_t)2 * waves * kTok4 * 4 * sizeof(float) : 0);
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
  const int threads = waves * kWave;
  const int resident = num_cus * wg_per_cu;
  int wgs_needed = 0;
  for (int i = 0; i < g.n_members; ++i) {
    const int blocks = g.task_end[i] - (i ? g.task_end[i - 1] : 0);
    wgs_needed += (blocks + blocks_per_wg - 1) / blocks_per_wg;
  }
  const int rounds = wgs_needed > resident ? (wgs_needed + resident - 1) / resident : 1;
  GroupDev gl = g;
  int grid = 0;
  for (int i = 0; i < g.n_members; ++i) {
    const int blocks = g.task_end[i] - (i ? g.task_end[i - 1] : 0);
    const int wg_i = ((blocks + blocks_per_wg - 1) / blocks_per_wg + rounds - 1) / rounds;
    grid += wg_i < 1 ? 1 : wg_i;
    gl.wg_end[i] = grid;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, stream, gl, kit, slices);
  return hipGetLastError();
}

// most token rows one launch can take for this shape (0: the route does not apply)
int quad_capacity(int M, int K, int rank, bool has_r) {
  for (int c = 16; c >= 1; c >>= 1)
    if (quad_supported(c, K, rank, has_r)) return c < M ? c : M;
  return 0;
}

hipError_t launch_quad(GroupDev& g, int num_cus, hipStream_t stream) {
  int total = 0;
  for (int i = 0; i < g.n_members; ++i) {
    total += (g.mem[i].N + kQuadRows - 1) / kQuadRows;
    g.task_end[i] = total;
  }
  const int kit = (g.K / 32 + kWave - 1) / kWave;
  const bool has_r = g.r != nullptr;
  const int lw = has_r ? quad_lw(g.rank, kit) : 0;
  const int tokens = quad_tokens(g.M);
  const size_t lds = quad_lds(tokens, g.K, has_r ? g.rank : 0).total;
  const bool wide = g.group_size >= 128;
#define GLOWQ_CASE(MM, LL)                                                                        \
  if (tokens == MM && lw == LL)                                                                   \
    return wide ? launch_quad_t<MM, LL, true>(g, kit, num_cus, lds, stream)                       \
                : launch_quad_t<MM, LL, false>(g, kit, num_cus, lds, stream);
#define GLOWQ_CASES(MM) GLOWQ_CASE(MM, 0) GLOWQ_CASE(MM, 2) GLOWQ_CASE(MM, 4)
  GLOWQ_CASES(1) GLOWQ_CASES(2) GLOWQ_CASES(4) GLOWQ_CASES(8) GLOWQ_CASES(16)
#undef GLOWQ_CASES
#undef GLOWQ_CASE
  return hipErrorInvalidValue;
}

}  // namespace glowq
