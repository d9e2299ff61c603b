// Tiled copy of a member's weights for the matrix-core kernels: a deterministic re-ordering of the canonical buffers
// (qweight [N, K/8] int32, scales, qzeros), written once at conversion time by glowq_pack_tiled, in which one coalesced
// 16-byte-per-lane load of a wave lands every lane's codes where v_mfma_f32_32x32x16_f16 wants its B operand.  The
// canonical buffers keep K contiguous per output row; the B operand wants 32 output rows side by side, so a kernel that
// reads them as they are has to send every byte through LDS once (written in memory order, read back in lane order).
//
//   row block rb = 32 consecutive output rows, super-block sb = 256 consecutive input columns = two halves g of 128
//   chunk(rb, sb) at byte (sb * RB + rb) * 4352 of the stream, RB = ceil(N / 32) -- super-block major: waves that walk K
//   in step read one contiguous window of the stream at a time, which the DRAM pages like better than a window per wave:
//     bytes [1024 j + 16 l, +16), j = 2 g + p (g, p in {0, 1}), lane l = 32 h + c:
//         the 16 bytes (4 words, 32 codes) at byte 64 g + 32 h + 16 p of the 128-byte segment sb of row 32 rb + c,
//         i.e. the codes of columns 256 sb + 128 g + 64 h + 32 p + [0, 32): word i of it feeds the matrix instruction
//         (g, p, i), whose sixteen k values (eight per lane half h) all lie in half g -- one quantisation group.
//         Inside a word the code of its column k (nibble k of the canonical word) sits in nibble (0,4,1,5,2,6,3,7)[k]:
//         the masks w & 0x000F000F, w & 0x00F000F0, (w >> 8) & 0x000F000F, (w >> 8) & 0x00F000F0 then yield the pairs of
//         columns (0,1), (2,3), (4,5), (6,7) in order, and the activations need no permutation
//     bytes [4096 + 8 c + 4 g, +4): low half = fp16 scale of (row 32 rb + c, the group of column 256 sb + 128 g),
//         high half = fp16(-zero-point * 2^-16) of the same group
//   rows past N hold zero codes, scale 0 and zero-point 0.
// Needs K % 256 == 0 and groups of 128 columns or a larger power of two (a half of 128 columns lies in one group).
//
// Tiled left factor (fp16 B operand of the correction blocks [r | L]): rank blocks jb of 64 columns, LB = ceil(rank / 64),
//   chunk(rb, jb) at byte (rb * LB + jb) * 4096: bytes [1024 t + 16 l, +16) = the eight values
//   L[32 rb + c, 64 jb + 32 h + 8 t + e], e = 0..7, those with e in {2, 3, 6, 7} multiplied by 16 (the kernels stage
//   r with those pairs divided by 16, as the raw-code kernel stages all its activations: skinny_tiled.hip); zero past
//   the rank and past N.
#pragma once

#include <stddef.h>

namespace glowq {
namespace tiled {

constexpr int kRows = 32;
constexpr int kSuper = 256;
constexpr int kCodeBytes = 4096;
constexpr int kSideBytes = 256;
constexpr int kChunk = kCodeBytes + kSideBytes;
constexpr int kLChunk = 4096;

inline bool applies(int K, int group_size) {
  return K > 0 && (K & (kSuper - 1)) == 0 && group_size >= 128 && (group_size & (group_size - 1)) == 0;
}
inline size_t weight_bytes(int N, int K) { return (size_t)((N + kRows - 1) / kRows) * (size_t)(K / kSuper) * kChunk; }
inline size_t left_bytes(int N, int rank) { return (size_t)((N + kRows - 1) / kRows) * (size_t)((rank + 63) / 64) * kLChunk; }

}  // namespace tiled
}  // namespace glowq
