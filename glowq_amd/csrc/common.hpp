// Shared device helpers for the gfx950 W4A16 + GlowQ kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/glowq_w4a16.h"

namespace glowq {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Device-side copy of one group member (pointers already typed).
struct MemberDev {
  const int32_t* qweight;
  const half_t* scales;
  const int32_t* qzeros;
  const half_t* L;
  const half_t* bias;
  half_t* y;
  const unsigned char* side;  // the member's side stream (side_stream.hpp) or nullptr
  int side_rank;              // the rank it was packed for
  const void* tiled;          // the member's tiled weights (tiled.hpp) or nullptr
  const void* tiled_L;        // its tiled left factor or nullptr
  int tiled_rank;             // the rank tiled_L was packed for
  int N, ldw, lds, ldz, ldy;
};

struct GroupDev {
  const half_t* x;  // [M, K]
  const half_t* r;  // [M, rank] or nullptr
  // set by the entry point that also produces r: the projection r_out = x R^T is launched ahead of the group
  const half_t* R;  // [rank, K] or nullptr
  half_t* r_out;
  void* ws;         // caller's workspace for the many-row projection (or nullptr) and its size
  size_t ws_bytes;
  // single-token stream GEMV with the projection inside the launch (run_group decides): the hand-over words of r, one
  // 64-bit word per entry, and the number of polls a reader spends on one before it computes the entry itself
  unsigned long long* pub;
  unsigned pub_spin;
  int pub_mute;
  MemberDev mem[GLOWQ_MAX_MEMBERS];
  int task_end[GLOWQ_MAX_MEMBERS];  // exclusive prefix of per-member task counts
  int wg_end[GLOWQ_MAX_MEMBERS];    // exclusive prefix of the workgroups assigned to each member
  int n_members;
  int M, K, group_size, rank;
  float alpha;
};

// Arguments of the chained single-token forms of the stream GEMV (stream_kernel.hpp).
namespace streamk {
constexpr int kAccCopies = GLOWQ_CHAIN_ACC_COPIES;
constexpr int kAccStride = GLOWQ_CHAIN_ACC_STRIDE;
constexpr int kProPlain = 0, kProAcc = 1, kProNormAcc = 2, kProProj = 3;
constexpr int kEpiNone = 0, kEpiResidual = 1, kEpiSwiglu = 2;

struct ChainDev {
  const half_t* norm_w;     // kProNormAcc: weight of the norm in front of this group [K]
  const long long* acc_in;  // kProAcc, kProNormAcc: accumulator the producer in front filled
  half_t* resid;            // kEpiResidual: residual stream rows of this group's output [N], read then written
  const half_t* next_w;     // kEpiResidual: weight of the norm that follows [N], or nullptr (all ones)
  const half_t* next_rt;    // epilogues: right factor of the group that follows, transposed [N, rank]; nullptr: no P
  long long* acc_out;       // with next_rt
  half_t* act;              // kEpiSwiglu: gated activations [N]
  float eps;                // kProNormAcc
  float part_limit;         // epilogues: see above
  // kProProj: right factor [rank, K], where r goes for the caller [rank], the hand-over words [rank], polls per word
  const half_t* proj_R;
  half_t* proj_r_out;
  unsigned long long* proj_pub;
  unsigned proj_spin;
  int proj_mute;  // producers keep their entries to themselves (a test of what readers do when no entry ever arrives)
};
}  // namespace streamk

// Records the calling thread's error message (returned by glowq_last_error) and hands back `code`.
int fail(int code, const char* fmt, ...);
// Compute units of the current device (cached).
int num_cus();
// Leaves the kernel a group launch used in the calling thread's launch record (glowq_last_launch): its name with the
// template arguments of the instantiation, grid and workgroup size.
void note_launch(int grid_x, int grid_y, int block, const char* fmt, ...);

// Raises a kernel's dynamic LDS limit to `bytes` on the current device when that is above the 48 KB default and above
// what this call site asked for before.  `raised` is the call site's own table (one slot per device); host threads may
// race on a slot, in which case the attribute is set more than once, to values that only grow.
struct LdsLimit {
  std::atomic<size_t> raised[64] = {};
};
inline hipError_t ensure_dynamic_lds(const void* kernel, size_t bytes, LdsLimit& site) {
  if (bytes <= 48 * 1024) return hipSuccess;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  if (bytes <= site.raised[dev].load(std::memory_order_acquire)) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return e;
  size_t seen = site.raised[dev].load(std::memory_order_relaxed);
  while (seen < bytes && !site.raised[dev].compare_exchange_weak(seen, bytes, std::memory_order_release)) {
  }
  return hipSuccess;
}

__device__ __forceinline__ uint32_t nibble(uint32_t word, int idx) { return (word >> (4 * idx)) & 0xFu; }

template <typename T>
__device__ __forceinline__ T bitcast_u32(uint32_t v) {
  return __builtin_bit_cast(T, v);
}

// Sum over the 64 lanes of a wave; every lane gets the total.  Four DPP steps reduce each row of
// 16 lanes, the four row totals are then combined through scalar lane reads.
__device__ __forceinline__ float wave_sum(float v) {
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
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
  return (a + b) + (c + d);
}

// Sum over the 4 lanes of a quad; every lane of the quad gets the total.
__device__ __forceinline__ float quad_sum(float v) {
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true);
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true);
  v += __builtin_bit_cast(float, t);
  return v;
}

// x * sigmoid(x) in fp32: one exponential and one reciprocal (the hardware approximations, about 1 ulp each: far inside
// the fp16 rounding that follows); a full-precision division costs ten instructions more per element.
__device__ __forceinline__ float silu_f32(float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

}  // namespace glowq
