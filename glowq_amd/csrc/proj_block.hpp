// r[m, j] = fp16(sum_k x[m, k] R[j, k]) for a block of kM token rows and kJ rows of R by the first 256 threads of a
// workgroup: the body of shared_proj_block_kernel (misc.hip), shared with the group kernels that compute r themselves
// in workgroups of their own in front of the grid.  Every 16-byte piece of x the workgroup loads meets kJ rows of R and
// every piece of R meets kM token rows.  K % 8 == 0, 16-byte aligned rows.
#pragma once

#include "common.hpp"

namespace glowq {

// part: 4 x kM x kJ floats of LDS.  `store(m, j, value)` is called by thread m * kJ + j of the team for the
// entries inside [M, rank].  A team is 256 threads, `tid` the thread's index in it: by default the first 256 threads of
// the workgroup (threads 256 and up must then not call this: the barrier inside counts the waves that arrive).  Several
// teams of one workgroup may each take a block of their own at the same time, with a `part` of their own; all of them
// then have to call this equally often, a team without a block with `active` false (it only meets the barrier).
template <int kM, int kJ, typename Store>
__device__ __forceinline__ void proj_block_body(const half_t* __restrict__ x, const half_t* __restrict__ R, int M, int K, int rank,
                                                int j0, int m0, float* part, Store&& store, int tid = (int)threadIdx.x,
                                                bool active = true) {
  if (!active) {
    __syncthreads();
    return;
  }
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  float acc[kM][kJ];
#pragma unroll
  for (int m = 0; m < kM; ++m)
#pragma unroll
    for (int j = 0; j < kJ; ++j) acc[m][j] = 0.f;
  const int words = K >> 3;
  constexpr int kBatch = (kM + kJ) > 8 ? 1 : 2;  // all loads of a batch are issued before the first is used
  const h8* xrow[kM];
  const h8* rrow[kJ];
#pragma unroll
  for (int m = 0; m < kM; ++m) xrow[m] = reinterpret_cast<const h8*>(x + (size_t)min(m0 + m, M - 1) * K);
#pragma unroll
  for (int j = 0; j < kJ; ++j) rrow[j] = reinterpret_cast<const h8*>(R + (size_t)min(j0 + j, rank - 1) * K);
  for (int w0 = tid; w0 < words; w0 += kBatch * 256) {
    h8 rv[kJ][kBatch], xv[kM][kBatch];
    float live[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int w = w0 + b * 256;
      live[b] = w < words ? 1.f : 0.f;
      const int wc = min(w, words - 1);
#pragma unroll
      for (int j = 0; j < kJ; ++j) rv[j][b] = rrow[j][wc];
#pragma unroll
      for (int m = 0; m < kM; ++m) xv[m][b] = xrow[m][wc];
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b)
#pragma unroll
      for (int m = 0; m < kM; ++m)
#pragma unroll
        for (int j = 0; j < kJ; ++j) {
          float d = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            d = __builtin_amdgcn_fdot2(h2{rv[j][b][2 * i], rv[j][b][2 * i + 1]}, h2{xv[m][b][2 * i], xv[m][b][2 * i + 1]}, d, false);
          acc[m][j] = __builtin_fmaf(live[b], d, acc[m][j]);
        }
  }
#pragma unroll
  for (int m = 0; m < kM; ++m)
#pragma unroll
    for (int j = 0; j < kJ; ++j) {
      const float v = wave_sum(acc[m][j]);
      if (lane == 0) part[wave * (kM * kJ) + m * kJ + j] = v;
    }
  __syncthreads();
  if (tid < kM * kJ) {
    const int m = m0 + tid / kJ, j = j0 + tid % kJ;
    if (m < M && j < rank)
      store(m, j, (part[tid] + part[kM * kJ + tid]) + (part[2 * kM * kJ + tid] + part[3 * kM * kJ + tid]));
  }
}

}  // namespace glowq
