// Tags for values that workgroups of one launch hand to each other through device memory (the group kernels that
// compute the shared projection themselves: stream_kernel.hpp, skinny.hip).  A tag names the launch: it is built from the
// dispatch id -- the position of the launch's packet in its hardware queue, which a replay of a captured graph renews
// like any other launch -- and from the address of that queue, with the top bit set so that zeroed memory never
// matches.  Words left by earlier launches therefore never pass for this launch's, and nothing has to be cleared.
#pragma once

#include "common.hpp"

namespace glowq {

extern "C" __device__ unsigned long long glowq_dispatch_id(void) __asm("llvm.amdgcn.dispatch.id");
constexpr unsigned long long kTagMask = 0xFFFFFFFFFFFFull;  // a tag takes the low 48 bits of a 64-bit word
__device__ __forceinline__ unsigned long long launch_tag() {
  const unsigned long long q = (unsigned long long)reinterpret_cast<uintptr_t>(__builtin_amdgcn_queue_ptr());
  return (glowq_dispatch_id() & 0xFFFFFFFull) | (((q >> 8) & 0x7FFFFull) << 28) | (1ull << 47);
}

// Of each eight workgroups at the head of a grid the first four take a role in front (producers of the handed-over
// values, collectors), the other four are ordinary workgroups like the rest: workgroup i runs on part i mod 8 of the
// chip, and parts 4..7 were seen to start a launch 1.1 to 1.5 us behind parts 0..3.  `wg` comes in as the workgroup's
// index in the grid and goes out as its index among the ordinary workgroups; the result is its role in front
// (0 .. front - 1; front and above: none to play), or -1 for an ordinary workgroup.
__device__ __forceinline__ int front_role(int& wg, int front) {
  const int zone = 2 * ((front + 3) & ~3);
  int role = -1;
  if (wg < zone) {
    if ((wg & 7) < 4) role = (wg >> 3) * 4 + (wg & 3);
    else wg = (wg >> 3) * 4 + (wg & 3);
  } else {
    wg -= zone >> 1;
  }
  return role;
}
// the grid of `ordinary` workgroups with `front` of them in front (a front padded to a multiple of four takes as many
// ordinary workgroups between it)
__host__ __device__ constexpr int front_grid(int ordinary, int front) {
  const int padded = (front + 3) & ~3;
  return ordinary > padded ? padded + ordinary : 2 * padded;
}

}  // namespace glowq
