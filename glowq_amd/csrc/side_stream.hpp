// Layout of a member's "side stream": the scales, zero-points and left-factor rows of every row block of two output
// rows, repacked into the order and the registers the single-token stream GEMV wants them in, so that a wave fetches
// them with one to three fully coalesced loads per row block instead of one small request per array and row.
// A deterministic function of the canonical buffers (scales [N, lds] fp16, qzeros [N, ldz] int32, L [N, rank] fp16);
// the canonical buffers stay what every other kernel reads.
//
// Row block b (rows 2b, 2b+1) owns `dwords` = np + 2 lw dwords per lane, 256 * dwords bytes:
//   dword p < np            lane 32 r + i: fp16 scale (bits 0-15) and zero-point (bits 16-19) of group
//                           min(gbase(p) + i, G - 1) of row 2b + r, gbase(p) = first group of step 2p
//   dword np + 2 j + r      lane l: halves 2 (l + 64 j), 2 (l + 64 j) + 1 of row 2b + r of L (zero past the rank, for a
//                           row past N, or without L)
// stored in chunks of four dwords (the last chunk 1..4), each chunk lane-major: chunk c starts 1024 c bytes into the
// block and gives lane l its dwords at l * 4 * size(c).
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace glowq {

struct SideLayout {
  int kit;        // steps of 2048 columns per row
  int np;         // pairs of steps
  int lw;         // dwords of a row of L per lane
  int dwords;     // per lane and row block
  int upg_shift;  // log2 of the 16-byte units per quantisation group
  int groups;     // quantisation groups per row
};

__host__ __device__ inline bool side_layout(int K, int group_size, int rank, SideLayout& s) {
  if (K <= 0 || (K & 31) != 0 || K > 9 * 2048) return false;
  if (group_size < 128 || (group_size & (group_size - 1)) != 0) return false;
  if (rank < 0 || (rank & 1) != 0 || rank > 256) return false;
  const int U = K >> 5;
  s.kit = (U + 63) >> 6;
  s.np = (s.kit + 1) >> 1;
  s.lw = (rank + 127) >> 7;
  s.dwords = s.np + 2 * s.lw;
  s.upg_shift = 0;
  while ((32 << s.upg_shift) < group_size) ++s.upg_shift;
  s.groups = (U + (1 << s.upg_shift) - 1) >> s.upg_shift;
  return true;
}

__host__ __device__ inline int side_gbase(const SideLayout& s, int p) { return (128 * p) >> s.upg_shift; }

__host__ __device__ inline size_t side_block_bytes(const SideLayout& s) { return (size_t)256 * s.dwords; }

// byte offset of dword d of lane l inside a row block
__host__ __device__ inline size_t side_dword_offset(const SideLayout& s, int d, int lane) {
  const int c = d >> 2;
  const int size = s.dwords - 4 * c < 4 ? s.dwords - 4 * c : 4;
  return (size_t)1024 * c + (size_t)lane * 4 * size + 4 * (d & 3);
}

}  // namespace glowq
