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
#include "common.hpp"

namespace glowq {

// Activation staging shared by every wave-dot instantiation.
//   xs  [M][4][U] units of 8 halves: quarter j of unit u holds x[32u + 8j + {0,4,1,5,2,6,3,7}]
//   sig [M][U]    float: 2^-24 * sum of the 32 activations of unit u
//   rs  [M][rank] halves (only when a correction is applied)
template <int kM>
__device__ __forceinline__ void stage_activations(const GroupDev& g, int U, h8* xs, float* sig, half_t* rs) {
  const int words = g.K >> 3;  // 8 halves each
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

template <int kM, int kRows>
__global__ __launch_bounds__(256) void gemv_wave_dot_kernel(const GroupDev g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int U = g.K >> 5;                 // 16-byte units per row
  const int upg = g.group_size >> 5;      // units per quantisation group
  h8* xs = reinterpret_cast<h8*>(smem);
  float* sig = reinterpret_cast<float*>(smem + (size_t)kM * g.K * sizeof(half_t));
  half_t* rs = reinterpret_cast<half_t*>(sig + kM * U);

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int total_tasks = g.task_end[g.n_members - 1];
  int task = blockIdx.x * waves_per_block + wave;

  stage_activations<kM>(g, U, xs, sig, rs);
  __syncthreads();

  const int iters = (U + kWave - 1) / kWave;
  for (; task < total_tasks; task += gridDim.x * waves_per_block) {
    int mi = 0;
    while (mi + 1 < g.n_members && task >= g.task_end[mi]) ++mi;
    const MemberDev& mem = g.mem[mi];
    const int n0 = (task - (mi ? g.task_end[mi - 1] : 0)) * kRows;

    float tot[kRows][kM];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int m = 0; m < kM; ++m) tot[r][m] = 0.f;

    const int32_t* wrow[kRows];
    const half_t* srow[kRows];
    const int32_t* zrow[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int n = min(n0 + r, mem.N - 1);
      wrow[r] = mem.qweight + (size_t)n * mem.ldw;
      srow[r] = mem.scales + (size_t)n * mem.lds;
      zrow[r] = mem.qzeros + (size_t)n * mem.ldz;
    }

#pragma unroll 2
    for (int it = 0; it < iters; ++it) {
      const int uraw = lane + it * kWave;
      const bool active = uraw < U;
      const int u = active ? uraw : U - 1;
      const int grp = u / upg;

      u32x4 wv[kRows];
      float sc[kRows];
      float zp[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        wv[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[r]) + u);
        const float s = (float)srow[r][grp];
        sc[r] = active ? s : 0.f;
        zp[r] = (float)nibble((uint32_t)zrow[r][grp >> 3], grp & 7);
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
          dot_word(wv[r].x, xq[0], accA, accB);
          dot_word(wv[r].y, xq[1], accA, accB);
          dot_word(wv[r].z, xq[2], accA, accB);
          dot_word(wv[r].w, xq[3], accA, accB);
          float v = __builtin_fmaf(accB, 0.0625f, accA);
          v = __builtin_fmaf(-zp[r], sg, v);
          tot[r][m] = __builtin_fmaf(sc[r], v, tot[r][m]);
        }
      }
    }

    // undo the 2^-24 of the subnormal trick, then the rank-r correction: alpha * L[n,:] . r[m,:]
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int m = 0; m < kM; ++m) tot[r][m] *= 0x1p24f;

    if (mem.L != nullptr && g.r != nullptr) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int n = min(n0 + r, mem.N - 1);
        const half_t* lrow = mem.L + (size_t)n * g.rank;
        float corr[kM];
#pragma unroll
        for (int m = 0; m < kM; ++m) corr[m] = 0.f;
        if ((g.rank & 1) == 0) {
          for (int jj = lane; jj < (g.rank >> 1); jj += kWave) {
            const h2 lp = reinterpret_cast<const h2*>(lrow)[jj];
#pragma unroll
            for (int m = 0; m < kM; ++m)
              corr[m] = __builtin_amdgcn_fdot2(lp, reinterpret_cast<const h2*>(rs + m * g.rank)[jj], corr[m], false);
          }
        } else {
          for (int jj = lane; jj < g.rank; jj += kWave) {
            const float lv = (float)lrow[jj];
#pragma unroll
            for (int m = 0; m < kM; ++m) corr[m] = __builtin_fmaf(lv, (float)rs[m * g.rank + jj], corr[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < kM; ++m) tot[r][m] = __builtin_fmaf(g.alpha, corr[m], tot[r][m]);
      }
    }

#pragma unroll
    for (int r = 0; r < kRows; ++r) {
#pragma unroll
      for (int m = 0; m < kM; ++m) {
        const float v = wave_sum(tot[r][m]);
        const int n = n0 + r;
        if (lane == 0 && n < mem.N) {
          const float b = mem.bias ? (float)mem.bias[n] : 0.f;
          mem.y[(size_t)m * mem.ldy + n] = (half_t)(v + b);
        }
      }
    }
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
  const size_t U = (size_t)K >> 5;
  return (size_t)M * K * sizeof(half_t) + (size_t)M * U * sizeof(float) + (has_r ? (size_t)M * rank * sizeof(half_t) : 0);
}

template <int kM, int kRows>
static hipError_t launch_wave_dot_t(const GroupDev& g, int grid, size_t lds, hipStream_t stream) {
  auto kern = gemv_wave_dot_kernel<kM, kRows>;
  static size_t configured = 48 * 1024;  // largest dynamic LDS size this instantiation was raised to
  if (lds > configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    configured = lds;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, g);
  return hipGetLastError();
}

// Rows per wave task for the wave-dot route: enough tasks to put several waves on every SIMD while
// keeping a few independent rows per wave for load-level parallelism.
int wave_dot_rows(long total_rows) {
  if (total_rows >= 16384) return 4;
  if (total_rows >= 4096) return 2;
  return 1;
}

hipError_t launch_wave_dot(GroupDev& g, int rows_per_task, int num_cus, hipStream_t stream) {
  int total = 0;
  for (int i = 0; i < g.n_members; ++i) {
    total += (g.mem[i].N + rows_per_task - 1) / rows_per_task;
    g.task_end[i] = total;
  }
  const size_t lds = wave_dot_lds_bytes(g.M, g.K, g.rank, g.r != nullptr);
  const int blocks_needed = (total + 3) / 4;
  // resident workgroups per CU: bounded by LDS (160 KB) and by 8 waves per SIMD
  int per_cu = (int)((160 * 1024) / (lds + 256));
  if (per_cu > 8) per_cu = 8;
  if (per_cu < 1) per_cu = 1;
  int grid = blocks_needed < num_cus * per_cu ? blocks_needed : num_cus * per_cu;
  if (grid < 1) grid = 1;
#define GLOWQ_CASE(MM, RR) \
  if (g.M == MM && rows_per_task == RR) return launch_wave_dot_t<MM, RR>(g, grid, lds, stream);
  GLOWQ_CASE(1, 1) GLOWQ_CASE(1, 2) GLOWQ_CASE(1, 4)
  GLOWQ_CASE(2, 1) GLOWQ_CASE(2, 2) GLOWQ_CASE(2, 4)
  GLOWQ_CASE(3, 1) GLOWQ_CASE(3, 2) GLOWQ_CASE(3, 4)
  GLOWQ_CASE(4, 1) GLOWQ_CASE(4, 2) GLOWQ_CASE(4, 4)
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
