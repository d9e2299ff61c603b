// Prefill GEMM for gfx950: y[M,N] = x[M,K] . deq(W)[N,K]^T (+ alpha * r[M,rank] . L[N,rank]^T) on fp16 MFMA
// with fp32 accumulation.
//
// A workgroup of 4 waves owns a BM x BN output tile (BM = 32*kMT rows, BN = 128*kNT columns); the waves
// split the columns, each holding kMT x kNT accumulator tiles of 32x32 (v_mfma_f32_32x32x16_f16).
//   * Activations go global -> registers -> LDS (double-buffered, rows padded to 144 bytes so that the
//     16-byte fragment reads of 32 consecutive rows fall into distinct banks) and are read back as MFMA
//     A fragments by all four waves.
//   * Weights never touch LDS or HBM as fp16: the B operand of the 32x32x16 MFMA wants, per lane, 8
//     consecutive k of one output column -- exactly one int32 word of 8 int4 codes.  A lane loads 16 bytes
//     (4 words = the 4 MFMA k-steps of a 64-deep block) and dequantises them in registers to
//     fp16((code - zero) * scale): the codes are masked into the mantissa of 1024.0 / 64.0, the offset
//     and zero-point are removed by one exact packed subtraction, and one packed multiply rounds once,
//     which is bit-identical to the reference's dequantisation.  Every weight is dequantised exactly once.
//   * The masks deliver the codes of a word in the order (0,4,1,5,2,6,3,7); the activations are permuted
//     the same way on their way into LDS, so no instruction is spent on reordering weights.
//   * The rank-r correction is a K-extension that runs first: acc = r . L^T on the same pipeline with an
//     fp16 B operand, acc *= alpha, then the quantised K loop accumulates on top.
#include <cstdlib>

#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "tiled.hpp"

namespace glowq {

constexpr int kBK = 64;              // k depth of one pipeline step
constexpr int kARow = kBK + 8;       // padded LDS row, in halves (144 bytes)

struct GemmArgs {
  const half_t* x;        // [M, K]
  const half_t* r;        // [M, rank] or nullptr
  const int32_t* qweight; // [N, ldw] (quantised B) or nullptr
  const half_t* scales;
  const int32_t* qzeros;
  const half_t* bmat;     // [N, ldb] fp16 B operand: L for the correction, or the whole B of a plain GEMM
  const half_t* bias;
  half_t* y;              // [M, ldy]
  const unsigned char* wt;  // the member's tiled weights (tiled.hpp) or nullptr
  const unsigned char* lt;  // its tiled left factor or nullptr
  int M, N, K, group_size, rank;
  int ldw, lds, ldz, ldb, ldy;
  float alpha;
};

// One launch covers every member of a group: workgroup b serves member i for blk_end[i-1] <= b < blk_end[i].
struct GemmGroup {
  GemmArgs m[GLOWQ_MAX_MEMBERS];
  int blk_end[GLOWQ_MAX_MEMBERS];
  int n;
  // split K (super-block form only): gridDim.y slices of whole super-blocks; every workgroup leaves its fp32 tile in
  // `partials` ([slice][tile][BM * BN] in accumulator-register order) and gemm_reduce_kernel adds them in slice order
  int slices;
  float* partials;
  // tail split (super-block form, slices == 1): workgroups [0, full) are whole tiles; behind them every tail tile comes
  // as tail_slices workgroups, slice t % tail_slices of tile full + t / tail_slices for t = blockIdx.x - full, which
  // leave partials ([slice][tail tile][BM * BN]) for gemm_reduce_kernel.  The last, partly filled round of workgroups
  // of a launch then costs its share of a round instead of a whole one.  tail_slices <= 1: off.
  int full, tail_slices;
};

__device__ __forceinline__ h8 permute_for_nibble_order(const h8& v) {
  h8 p;
  p[0] = v[0]; p[1] = v[4]; p[2] = v[1]; p[3] = v[5];
  p[4] = v[2]; p[5] = v[6]; p[6] = v[3]; p[7] = v[7];
  return p;
}

// 8 codes of one word -> fp16((code - zero) * scale), in nibble order (0,4,1,5,2,6,3,7).
// zb_lo = -(1024 + zero), zb_hi = -(64 + zero), both exact in fp16.
__device__ __forceinline__ h8 dequant_word(uint32_t w, h2 zb_lo, h2 zb_hi, h2 s2) {
  // the two exponent patterns (1024.0 and 64.0 in both halves) live in vector registers: with the nibble mask as the one
  // scalar operand the mask-and-merge is then a single v_and_or_b32 instead of an AND and an OR
  uint32_t e1024, e64;
  asm("v_mov_b32 %0, 0x64006400" : "=v"(e1024));
  asm("v_mov_b32 %0, 0x54005400" : "=v"(e64));
  const uint32_t hi = w >> 8;
  const h2 q0 = bitcast_u32<h2>((w & 0x000F000Fu) | e1024);
  const h2 q1 = bitcast_u32<h2>((w & 0x00F000F0u) | e64);
  const h2 q2 = bitcast_u32<h2>((hi & 0x000F000Fu) | e1024);
  const h2 q3 = bitcast_u32<h2>((hi & 0x00F000F0u) | e64);
  const h2 d0 = (q0 + zb_lo) * s2;
  const h2 d1 = (q1 + zb_hi) * s2;
  const h2 d2 = (q2 + zb_lo) * s2;
  const h2 d3 = (q3 + zb_hi) * s2;
  h8 out;
  out[0] = d0[0]; out[1] = d0[1]; out[2] = d1[0]; out[3] = d1[1];
  out[4] = d2[0]; out[5] = d2[1]; out[6] = d3[0]; out[7] = d3[1];
  return out;
}

// kQuant: B is the int4 weight (with the optional correction phase in front); otherwise B is plain fp16.
// kSuper (quantised B, K % 256 == 0, group sizes of 128 and up): the K loop walks 256-column super-blocks in which lane
// (column c, half h) owns the 64 contiguous bytes of codes [256 sb + 128 h, +128) of its weight row -- one quantisation
// group, one scale and zero-point per super-block -- and the weights reach the B operand through a wave-private LDS tile
// that is filled in memory order (8 lanes per 128-byte row segment).  Fragment loads straight from memory, one 16-byte
// request per lane and cache line, make every request pull a whole line out of L2.
template <int kMT, int kNT, bool kQuant, bool kSuper = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((kMT * kNT >= 16 ? 1 : 2), (kMT * kNT >= 16 ? 1 : 8))))
void gemm_mfma_kernel(const GemmGroup gg, const int m_blocks) {
  // member of this workgroup, picked with scalar selects from fixed kernel-argument offsets
  // which tile and which slice of its K range this workgroup serves
  int wg = (int)blockIdx.x, slice = (int)blockIdx.y, nslices = gg.slices, part_tile = (int)blockIdx.x, part_tiles = (int)gridDim.x;
  if (kQuant && kSuper && gg.tail_slices > 1) {
    nslices = 1;
    if (wg >= gg.full) {
      const int t = wg - gg.full;
      part_tile = t / gg.tail_slices;
      slice = t - part_tile * gg.tail_slices;
      wg = gg.full + part_tile;
      nslices = gg.tail_slices;
      part_tiles = ((int)gridDim.x - gg.full) / gg.tail_slices;
    }
  }
  GemmArgs a = gg.m[0];
  int blk_base = 0;
#define GLOWQ_PICK(i)                                         \
  if (gg.n > i && wg >= gg.blk_end[i - 1]) {                 \
    a = gg.m[i];                                              \
    blk_base = gg.blk_end[i - 1];                             \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int BM = 32 * kMT;
  constexpr int BN = 128 * kNT;
  half_t* lds_a = reinterpret_cast<half_t*>(smem);  // [2][BM][kARow]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int blk = wg - blk_base;
  const int bm = blk % m_blocks;  // row blocks vary fastest: neighbouring workgroups share weight columns
  const int bn = blk / m_blocks;
  const int m0 = bm * BM;
  const int ln = lane & 31;  // column inside a 32-wide tile (B operand, accumulator) / row inside a tile (A operand)
  const int lh = lane >> 5;  // which half of the k range of an MFMA step this lane feeds

  int ncol[kNT];  // weight row (= output column) this lane feeds, clamped for loads
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) ncol[tn] = min(bn * BN + wave * (32 * kNT) + tn * 32 + ln, a.N - 1);

  f16v acc[kMT][kNT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tm][tn][i] = 0.f;

  // ---- activation tile: global -> registers -> LDS ------------------------------------------------
  // BM rows x 8 octets (16 bytes); thread t takes octets t, t+256, ...: 8 consecutive threads read the
  // 128 contiguous bytes of one row.
  struct ARegs {
    u32x4 v[kMT];
  };
  ARegs areg, areg1;
  auto load_a_to = [&](ARegs& dst, const half_t* src, int ld, int kb) {
#pragma unroll
    for (int i = 0; i < kMT; ++i) {
      const int q = tid + 256 * i;
      const int row = min(m0 + (q >> 3), a.M - 1);
      dst.v[i] = *reinterpret_cast<const u32x4*>(src + (size_t)row * ld + kb + (q & 7) * 8);
    }
  };
  auto store_a_from = [&](const ARegs& srcr, int stage, bool permute) {
#pragma unroll
    for (int i = 0; i < kMT; ++i) {
      const int q = tid + 256 * i;
      half_t* dst = lds_a + ((size_t)stage * BM + (q >> 3)) * kARow + (q & 7) * 8;
      const h8 v = __builtin_bit_cast(h8, srcr.v[i]);
      *reinterpret_cast<h8*>(dst) = permute ? permute_for_nibble_order(v) : v;
    }
  };
  auto store_a = [&](int stage, bool permute) { store_a_from(areg, stage, permute); };
  // A fragment of MFMA step t for row tile tm: octet (4*lh + t) of row tm*32 + ln
  auto read_a = [&](int stage, int tm, int t) {
    const half_t* src = lds_a + ((size_t)stage * BM + tm * 32 + ln) * kARow + (4 * lh + t) * 8;
    return *reinterpret_cast<const h8*>(src);
  };
  auto mma_step = [&](int stage, const h8 (&bfrag)[kNT][4]) {
    constexpr int kChunk = kMT < 4 ? kMT : 4;  // row tiles whose A fragments are live at once
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int c = 0; c < kMT; c += kChunk) {
        h8 af[kChunk];
#pragma unroll
        for (int i = 0; i < kChunk; ++i) af[i] = read_a(stage, c + i, t);
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < kChunk; ++i)
            acc[c + i][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bfrag[tn][t], acc[c + i][tn], 0, 0, 0);
      }
    }
  };

  int stage = 0;

  // ---- phase 1: the correction as a K-extension, acc = r . L^T, fp16 B operand ----------------------
  if (kQuant && a.r != nullptr && slice == 0) {
    // ranks are multiples of 8: in a partial last block the octets of r past the rank count as zero and L is read
    // from the row's last octet (finite values)
    const int steps = (a.rank + kBK - 1) / kBK;
    auto load_r = [&](int kb) {
#pragma unroll
      for (int i = 0; i < kMT; ++i) {
        const int q = tid + 256 * i;
        const int row = min(m0 + (q >> 3), a.M - 1);
        const int k = kb + (q & 7) * 8;
        const u32x4 v = *reinterpret_cast<const u32x4*>(a.r + (size_t)row * a.rank + min(k, a.rank - 8));
        areg.v[i] = k < a.rank ? v : u32x4{0u, 0u, 0u, 0u};
      }
    };
    load_r(0);
    store_a(stage, false);
    __syncthreads();
    for (int ks = 0; ks < steps; ++ks) {
      h8 bfrag[kNT][4];
      if constexpr (kSuper) {
        // the wave's 32 kNT rows of L, 128 bytes of this block each, in memory order (8 lanes per row) through its LDS
        // tile, as the weights of the main loop: fragment loads straight from memory cost a line per lane
        unsigned char* ltile = smem + (size_t)2 * BM * kARow * sizeof(half_t) + (size_t)wave * (32 * kNT) * 144;
        u32x4 lreg[kNT * 4];
#pragma unroll
        for (int q = 0; q < kNT * 4; ++q)
          lreg[q] = *reinterpret_cast<const u32x4*>(a.bmat + (size_t)min(bn * BN + wave * (32 * kNT) + q * 8 + (lane >> 3), a.N - 1) * a.ldb +
                                                    min(ks * kBK + (lane & 7) * 8, a.rank - 8));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous block are done
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int q = 0; q < kNT * 4; ++q)
          *reinterpret_cast<u32x4*>(ltile + (q * 8 + (lane >> 3)) * 144 + (lane & 7) * 16) = lreg[q];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            bfrag[tn][t] = *reinterpret_cast<const h8*>(ltile + (tn * 32 + ln) * 144 + lh * 64 + t * 16);
      } else {
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            bfrag[tn][t] = *reinterpret_cast<const h8*>(a.bmat + (size_t)ncol[tn] * a.ldb + min(ks * kBK + 32 * lh + 8 * t, a.rank - 8));
      }
      if (ks + 1 < steps) load_r((ks + 1) * kBK);
      mma_step(stage, bfrag);
      if (ks + 1 < steps) store_a(stage ^ 1, false);
      __syncthreads();
      stage ^= 1;
    }
    if (a.alpha != 1.0f) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[tm][tn][i] *= a.alpha;
    }
  }

  // ---- phase 2: the main K loop ---------------------------------------------------------------------
  const int steps = a.K / kBK;
  const int gs_shift = __builtin_ctz(a.group_size);  // group sizes on this route are powers of two
  if constexpr (kQuant && kSuper) {
    // Sub-step ks = 4 sb + j covers columns {256 sb + 128 h + 32 j + [0, 32) : h = 0, 1}; the activation stage keeps
    // its [BM][64] shape with octets 0-3 = half 0 and octets 4-7 = half 1, so the fragment reads do not change.
    constexpr int kSeg = 144;  // bytes per row segment in the weight tile: 128 + 16, conflict-free fragment reads
    unsigned char* btile = smem + (size_t)2 * BM * kARow * sizeof(half_t) + (size_t)wave * (32 * kNT) * kSeg;
    // Every load of the loop is a buffer load: a uniform descriptor and a uniform byte offset that advances per step
    // (scalar registers) plus a 32-bit byte offset that a lane computes once.  With 64-bit addresses per lane and load
    // the address pairs alone spill the register file of the large tiles, and every reload of a spilled pair waits
    // for all loads in flight.  (The host keeps tensors whose byte extent does not fit 32 bits off this route.)
    const auto rsrc = [](const void* p, size_t bytes) {
      return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t rs_x = rsrc(a.x, (size_t)a.M * a.K * 2);
    const __amdgpu_buffer_rsrc_t rs_w = rsrc(a.qweight, ((size_t)(a.N - 1) * a.ldw + (a.K >> 3)) * 4);
    const __amdgpu_buffer_rsrc_t rs_s = rsrc(a.scales, ((size_t)(a.N - 1) * a.lds + (a.K >> gs_shift)) * 2);
    const __amdgpu_buffer_rsrc_t rs_z = rsrc(a.qzeros, ((size_t)(a.N - 1) * a.ldz + (((a.K >> gs_shift) + 7) >> 3)) * 4);
    uint32_t a_off[kMT], b_off[kNT * 4], s_off[kNT], z_off[kNT];
#pragma unroll
    for (int i = 0; i < kMT; ++i) {
      const int q = tid + 256 * i;
      const int oct = q & 7;
      a_off[i] = ((uint32_t)min(m0 + (q >> 3), a.M - 1) * (uint32_t)a.K + (oct >> 2) * 128 + (oct & 3) * 8) * 2u;
    }
#pragma unroll
    for (int q = 0; q < kNT * 4; ++q)
      b_off[q] = ((uint32_t)min(bn * BN + wave * (32 * kNT) + q * 8 + (lane >> 3), a.N - 1) * (uint32_t)a.ldw + (lane & 7) * 4) * 4u;
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) {
      s_off[tn] = (uint32_t)ncol[tn] * (uint32_t)a.lds * 2u;
      z_off[tn] = (uint32_t)ncol[tn] * (uint32_t)a.ldz * 4u;
    }
    auto load_a_sub = [&](ARegs& dst, int ks) {
      const int kc = min(ks, steps - 1);
      const int step_off = ((kc >> 2) * 256 + (kc & 3) * 32) * 2;
#pragma unroll
      for (int i = 0; i < kMT; ++i) dst.v[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, (int)a_off[i], step_off, 0);
    };
    struct BLoad {
      u32x4 w[kNT * 4];  // a super-block of the wave's 32 kNT weight rows in load order: row 8 q + lane / 8, piece lane % 8
      uint32_t s[kNT], z[kNT];
    };
    uint32_t cur_s[kNT], cur_z[kNT];
    auto issue_b = [&](int sb, BLoad& bl) {
      const int sbc = min(sb, (steps >> 2) - 1);
      const uint32_t grp = (uint32_t)((sbc * 256 + lh * 128) >> gs_shift);
#pragma unroll
      for (int q = 0; q < kNT * 4; ++q) bl.w[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (int)b_off[q], sbc * 128, 0);
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        bl.s[tn] = (uint32_t)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rs_s, (int)(s_off[tn] + grp * 2u), 0, 0);
        bl.z[tn] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs_z, (int)(z_off[tn] + (grp >> 3) * 4u), 0, 0);
      }
    };
    auto stage_b = [&](const BLoad& bl) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous super-block are done
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < kNT * 4; ++q)
        *reinterpret_cast<u32x4*>(btile + (q * 8 + (lane >> 3)) * kSeg + (lane & 7) * 16) = bl.w[q];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        cur_s[tn] = bl.s[tn];
        cur_z[tn] = bl.z[tn];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    BLoad bl;
    // j is a compile-time constant at every call site (the loop below is unrolled by four)
    auto step = [&](int ks, int j, ARegs& a_fill, const ARegs& a_store) {
      const int sb = ks >> 2;
      if (j == 0) stage_b(bl);
      const int grp = (sb * 256 + lh * 128) >> gs_shift;
      u32x4 raw[kNT];
      h2 zb_lo[kNT], zb_hi[kNT], s2[kNT];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        const half_t z = (half_t)(float)nibble(cur_z[tn], grp & 7);
        const half_t zl = (half_t)(-1024.0f) - z, zh = (half_t)(-64.0f) - z;
        zb_lo[tn] = h2{zl, zl};
        zb_hi[tn] = h2{zh, zh};
        s2[tn] = bitcast_u32<h2>(cur_s[tn] | (cur_s[tn] << 16));
        raw[tn] = *reinterpret_cast<const u32x4*>(btile + (tn * 32 + ln) * kSeg + lh * 64 + j * 16);
      }
      load_a_sub(a_fill, ks + 2);
      if (j == 0) issue_b(sb + 1, bl);  // behind the activation loads: waiting for those leaves the weights in flight
      // one code word per MFMA step is dequantised right before its MFMAs: 8 fragment registers live instead of 32
      constexpr int kChunk = kMT < 4 ? kMT : 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        h8 bf[kNT];
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn) bf[tn] = dequant_word(raw[tn][t], zb_lo[tn], zb_hi[tn], s2[tn]);
#pragma unroll
        for (int c = 0; c < kMT; c += kChunk) {
          h8 af[kChunk];
#pragma unroll
          for (int i = 0; i < kChunk; ++i) af[i] = read_a(stage, c + i, t);
#pragma unroll
          for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
            for (int i = 0; i < kChunk; ++i)
              acc[c + i][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[tn], acc[c + i][tn], 0, 0, 0);
        }
      }
      store_a_from(a_store, stage ^ 1, true);
      __syncthreads();
      stage ^= 1;
    };
    // this workgroup's super-blocks: all of them, or slice `slice` of `nslices`
    const int sb_total = steps >> 2;  // steps is a multiple of 4 here
    const int sb_per = (sb_total + nslices - 1) / nslices;
    const int ks0 = min(slice * sb_per, sb_total) * 4;
    const int ks1 = min(ks0 + sb_per * 4, steps);
    load_a_sub(areg, ks0);
    issue_b(ks0 >> 2, bl);
    load_a_sub(areg1, ks0 + 1);
    store_a_from(areg, stage, true);
    __syncthreads();
    for (int ks = ks0; ks < ks1; ks += 4) {
      step(ks, 0, areg, areg1);
      step(ks + 1, 1, areg1, areg);
      step(ks + 2, 2, areg, areg1);
      step(ks + 3, 3, areg1, areg);
    }
  } else if constexpr (kQuant) {
    // quantised B: per step and column tile one 16-byte load of codes, one scale, one zero-point word.
    // Two register sets alternate (no copies), and the prefetch of the next step is unconditional (the
    // last step re-reads its own block): a uniform number of loads per step keeps the wait counts exact,
    // so the loads issued at the top of a step stay in flight under that step's MFMAs.
    struct WRegs {  // all members 32-bit wide: the struct stays in registers
      u32x4 w[kNT];
      uint32_t s[kNT];  // fp16 bits of the scale
      uint32_t z[kNT];
    };
    auto load_w = [&](int kb, WRegs& wr) {
      const int grp = (kb + 32 * lh) >> gs_shift;
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        wr.w[tn] = *reinterpret_cast<const u32x4*>(a.qweight + (size_t)ncol[tn] * a.ldw + (kb >> 3) + 4 * lh);
        wr.s[tn] = reinterpret_cast<const unsigned short*>(a.scales)[(size_t)ncol[tn] * a.lds + grp];
        wr.z[tn] = (uint32_t)a.qzeros[(size_t)ncol[tn] * a.ldz + (grp >> 3)];
      }
    };
    // Step s: dequantise W(s) out of its register set, refill that set with W(s+2) and the matching
    // activation set with A(s+2), run the MFMAs of step s on LDS stage s%2, then move A(s+1) (loaded one
    // step ago, so it has had a whole step to arrive) into the other LDS stage.  Loads are unconditional
    // (clamped to the last block) so that every step issues the same number of them.
    auto step = [&](int ks, WRegs& wr, ARegs& a_fill, const ARegs& a_store) {
      const int kb = ks * kBK;
      h8 bfrag[kNT][4];
      const int grp = (kb + 32 * lh) >> gs_shift;
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        const half_t z = (half_t)(float)nibble(wr.z[tn], grp & 7);
        const half_t zl = (half_t)(-1024.0f) - z, zh = (half_t)(-64.0f) - z;
        const h2 zb_lo = {zl, zl}, zb_hi = {zh, zh};
        const h2 s2 = bitcast_u32<h2>(wr.s[tn] | (wr.s[tn] << 16));
        bfrag[tn][0] = dequant_word(wr.w[tn].x, zb_lo, zb_hi, s2);
        bfrag[tn][1] = dequant_word(wr.w[tn].y, zb_lo, zb_hi, s2);
        bfrag[tn][2] = dequant_word(wr.w[tn].z, zb_lo, zb_hi, s2);
        bfrag[tn][3] = dequant_word(wr.w[tn].w, zb_lo, zb_hi, s2);
      }
      const int kb2 = min(ks + 2, steps - 1) * kBK;
      load_w(kb2, wr);
      load_a_to(a_fill, a.x, a.K, kb2);
      mma_step(stage, bfrag);
      store_a_from(a_store, stage ^ 1, true);
      __syncthreads();
      stage ^= 1;
    };
    WRegs w0, w1;
    load_a_to(areg, a.x, a.K, 0);
    load_w(0, w0);
    load_a_to(areg1, a.x, a.K, min(1, steps - 1) * kBK);
    load_w(min(1, steps - 1) * kBK, w1);
    store_a_from(areg, stage, true);
    __syncthreads();
    for (int ks = 0; ks < steps; ks += 2) {
      step(ks, w0, areg, areg1);
      if (ks + 1 >= steps) break;
      step(ks + 1, w1, areg1, areg);
    }
  } else {
    // plain fp16 B (the shared projection r = x R^T for many rows): same two-deep pipeline, the B
    // fragments are loaded as they are (4 x 16 bytes per lane, column tile and step)
    struct BRegs {
      u32x4 v[kNT][4];
    };
    auto load_b = [&](int kb, BRegs& br) {
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          br.v[tn][t] = *reinterpret_cast<const u32x4*>(a.bmat + (size_t)ncol[tn] * a.ldb + kb + 32 * lh + 8 * t);
    };
    auto step = [&](int ks, BRegs& br, ARegs& a_fill, const ARegs& a_store) {
      h8 bfrag[kNT][4];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int t = 0; t < 4; ++t) bfrag[tn][t] = __builtin_bit_cast(h8, br.v[tn][t]);
      const int kb2 = min(ks + 2, steps - 1) * kBK;
      load_b(kb2, br);
      load_a_to(a_fill, a.x, a.K, kb2);
      mma_step(stage, bfrag);
      store_a_from(a_store, stage ^ 1, false);
      __syncthreads();
      stage ^= 1;
    };
    BRegs b0, b1;
    load_a_to(areg, a.x, a.K, 0);
    load_b(0, b0);
    load_a_to(areg1, a.x, a.K, min(1, steps - 1) * kBK);
    load_b(min(1, steps - 1) * kBK, b1);
    store_a_from(areg, stage, false);
    __syncthreads();
    for (int ks = 0; ks < steps; ks += 2) {
      step(ks, b0, areg, areg1);
      if (ks + 1 >= steps) break;
      step(ks + 1, b1, areg1, areg);
    }
  }

  // ---- epilogue: accumulator register i of a 32x32 tile is row 8*(i/4) + 4*lh + i%4, column ln ---------
  if constexpr (kQuant && kSuper) {
    if (nslices > 1) {
      float* part = gg.partials + ((size_t)slice * part_tiles + part_tile) * (BM * BN);
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < 16; ++i) part[((tm * kNT + tn) * 16 + i) * 256 + tid] = acc[tm][tn][i];
      return;
    }
  }
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) {
    const int n = bn * BN + wave * (32 * kNT) + tn * 32 + ln;
    if (n >= a.N) continue;
    const float b = a.bias ? (float)a.bias[n] : 0.f;
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + tm * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < a.M) a.y[(size_t)m * a.ldy + n] = (half_t)(acc[tm][tn][i] + b);
      }
    }
  }
}

// ---- the same GEMM on the tiled copy of the weights (tiled.hpp) ---------------------------------------------------
// Same tiles, same workgroup -> tile map, same split of K, same partial tiles and epilogue as gemm_mfma_kernel's
// super-block form, same arithmetic (the weight is rounded to fp16 once).  What differs is how the operands arrive:
//   * B: a wave's 16-byte loads of a chunk of the tiled stream ARE the B operands of its 32 x 256 block, in lane order;
//     scale and zero-point ride in the same chunk (one 8-byte load per lane and super-block).  No pass of the weights
//     through LDS, no gathers of scales and zero-point words, no per-wave barriers around a staging tile.  One set of
//     registers holds a super-block; each 16-byte piece is refilled with the next super-block's as soon as its four
//     words have been dequantised, a whole super-block of matrix instructions ahead of its use.
//   * A: the tiled copy holds the nibbles of a code word in the order in which the masks deliver them, so the
//     activations need no permutation and go from memory straight into LDS (buffer_load ... lds: no registers, no
//     vector instructions, no ds_write).  Stages of 128 columns (one quantisation-group half of a super-block)
//     instead of 64: half the barriers per matrix instruction.  A load of a wave fills one contiguous kilobyte of
//     LDS -- four rows of 256 bytes, no padding -- so bank conflicts are avoided by the choice of what goes where:
//     slot c' of row r holds the 16-byte piece c' ^ (r % 16) of that row, and a fragment read of piece c looks in
//     slot c ^ (r % 16): sixteen consecutive rows land in sixteen different slots.
//   * The correction runs first as before, with the tiled left factor as B operand (its pairs at positions 2, 3, 6, 7
//     of every octet are stored times 16, so r is staged through registers with those pairs divided by 16).
constexpr int kTRow = 256;  // bytes of a staged row: 128 halves, swizzled instead of padded
#ifndef GLOWQ_GDBG
#define GLOWQ_GDBG 0
#endif

// kWk = 2: eight waves on the same tile, the second four take the second half of the workgroup's K range with LDS stages
// of their own, and the two accumulator sets meet in LDS before the epilogue.  For launches with about one tile per
// compute unit: a SIMD then holds two waves of the one workgroup it has, instead of one wave with nothing to overlap its
// waits with, and the K loop of a tile takes half as many steps.
template <int kMT, int kNT, int kWk>
__global__ __launch_bounds__(256 * kWk) __attribute__((amdgpu_waves_per_eu((kMT * kNT >= 16 ? 1 : 2), (kMT * kNT >= 16 ? 1 : 8))))
void gemm_tiled_kernel(const GemmGroup gg, const int m_blocks) {
  int wg = (int)blockIdx.x, slice = (int)blockIdx.y, nslices = gg.slices, part_tile = (int)blockIdx.x, part_tiles = (int)gridDim.x;
  if (gg.tail_slices > 1) {
    nslices = 1;
    if (wg >= gg.full) {
      const int t = wg - gg.full;
      part_tile = t / gg.tail_slices;
      slice = t - part_tile * gg.tail_slices;
      wg = gg.full + part_tile;
      nslices = gg.tail_slices;
      part_tiles = ((int)gridDim.x - gg.full) / gg.tail_slices;
    }
  }
  GemmArgs a = gg.m[0];
  int blk_base = 0;
#define GLOWQ_PICK(i)                                         \
  if (gg.n > i && wg >= gg.blk_end[i - 1]) {                 \
    a = gg.m[i];                                              \
    blk_base = gg.blk_end[i - 1];                             \
  }
  GLOWQ_PICK(1)
  GLOWQ_PICK(2)
  GLOWQ_PICK(3)
#undef GLOWQ_PICK
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_all[];
  constexpr int BM = 32 * kMT;
  constexpr int BN = 128 * kNT;
  constexpr int kAL = 2 * kMT;  // 16-byte pieces of a stage (BM rows x 256 bytes) per thread
  static_assert(kWk == 1 || kWk == 2, "one or two K groups");
  const int gk = kWk > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;  // K group of this wave
  unsigned char* smem = smem_all + (size_t)gk * 2 * BM * kTRow;
  const int tid = (int)threadIdx.x & 255;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = wg - blk_base;
  const int bm = blk % m_blocks;  // row blocks vary fastest: neighbouring workgroups share weight columns
  const int bn = blk / m_blocks;
  const int m0 = bm * BM;
  const int ln = lane & 31, lh = lane >> 5;

  f16v acc[kMT][kNT];
#pragma unroll
  for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tm][tn][i] = 0.f;

  const auto rsrc = [](const void* p, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
  };
  const int RB = (a.N + 31) >> 5;
  const int SB = a.K >> 8;
  // row block of column tile tn of this wave, clamped into the member (columns past N are computed and dropped)
  int rb[kNT];
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) rb[tn] = min(bn * (BN / 32) + wave * kNT + tn, RB - 1);

  // ---- activations: piece q of thread t fills slot (t & 15) of row 16 q + (t >> 4) of the stage, which holds the
  // 16-byte piece (t & 15) ^ (row % 16) of that row's 256 bytes (row % 16 = (t >> 4) % 16 for every q)
  const int srow = tid >> 4;                    // 0..15: the row within a block of sixteen
  const int spiece = (tid & 15) ^ srow;         // the piece of the row this thread moves
  uint32_t a_row[kAL];
#pragma unroll
  for (int q = 0; q < kAL; ++q) a_row[q] = (uint32_t)min(m0 + srow + 16 * q, a.M - 1);
  // A fragment of row tile tm, piece c of the staged row (which 16 columns: see the callers)
  auto read_a = [&](int stage, int tm, int c) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(smem + (size_t)stage * BM * kTRow + (tm * 32 + ln) * kTRow + ((c ^ (ln & 15)) << 4));
  };

  int stage = 0;
  constexpr int kChunk = kMT < 4 ? kMT : 4;  // row tiles whose A fragments are live at once

  // ---- phase 1: the correction, acc = r . L^T, 128 rank columns (two blocks of the tiled left factor) per stage ----------
  if (a.r != nullptr && a.lt != nullptr && slice == 0) {
    const int LB = (a.rank + 63) >> 6;
    const __amdgpu_buffer_rsrc_t rs_r = rsrc(a.r, (size_t)a.M * a.rank * 2);
    const __amdgpu_buffer_rsrc_t rs_l = rsrc(a.lt, gk == 0 ? (size_t)RB * LB * tiled::kLChunk : 0);  // one K group adds the correction
    const int steps = (a.rank + 127) >> 7;
    u32x4 areg[kAL];
    auto load_r = [&](int st) __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < kAL; ++q) {
        // columns past the rank meet zeros of the left factor
        const uint32_t col = (uint32_t)st * 128u + (uint32_t)spiece * 8u;
        areg[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_r, (int)((a_row[q] * (uint32_t)a.rank + min(col, (uint32_t)a.rank - 8u)) * 2u), 0, 0);
        if (col >= (uint32_t)a.rank) areg[q] = u32x4{0u, 0u, 0u, 0u};
      }
    };
    auto store_r = [&](int stg) __attribute__((always_inline)) {
      unsigned char* dst = smem + (size_t)stg * BM * kTRow + srow * kTRow + (tid & 15) * 16;
      const h2 k16 = {(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
      for (int q = 0; q < kAL; ++q) {
        u32x4 o = areg[q];
        o.y = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.y) * k16);
        o.w = __builtin_bit_cast(uint32_t, bitcast_u32<h2>(o.w) * k16);
        *reinterpret_cast<u32x4*>(dst + 16 * q * kTRow) = o;
      }
    };
    load_r(0);
    store_r(stage);
    __syncthreads();
    for (int st = 0; st < steps; ++st) {
      u32x4 lf[kNT][2][4];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int jb = 2 * st + q;
          // a block past the rank: an offset past the end of the descriptor (zeros)
          const uint32_t base = jb < LB ? (uint32_t)(rb[tn] * LB + jb) * (uint32_t)tiled::kLChunk : 0xFFFF0000u;
#pragma unroll
          for (int t = 0; t < 4; ++t) lf[tn][q][t] = __builtin_amdgcn_raw_buffer_load_b128(rs_l, lane * 16 + t * 1024, (int)base, 0);
        }
      if (st + 1 < steps) load_r(st + 1);
#pragma unroll
      for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int c = 0; c < kMT; c += kChunk) {
            h8 af[kChunk];
#pragma unroll
            for (int i = 0; i < kChunk; ++i) af[i] = read_a(stage, c + i, 8 * q + 4 * lh + t);
#pragma unroll
            for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
              for (int i = 0; i < kChunk; ++i)
                acc[c + i][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], __builtin_bit_cast(h8, lf[tn][q][t]), acc[c + i][tn], 0, 0, 0);
          }
      if (st + 1 < steps) store_r(stage ^ 1);
      __syncthreads();
      stage ^= 1;
    }
    if (a.alpha != 1.0f) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[tm][tn][i] *= a.alpha;
    }
  }

  // ---- phase 2: the quantised K loop, a half of a super-block (128 columns, one quantisation group) per stage --------
  {
    const __amdgpu_buffer_rsrc_t rs_x = rsrc(a.x, (size_t)a.M * a.K * 2);
    // this workgroup's super-blocks: all of them, or slice `slice` of `nslices`; dealt to the K groups in contiguous halves.
    // Both groups run the same number of steps (they share the barriers): a step past a group's part reads past the end of
    // its descriptor -- zero codes at scale zero.
    const int sb_per = (SB + nslices - 1) / nslices;
    const int ws0 = min(slice * sb_per, SB), ws1 = min(ws0 + sb_per, SB);
    const int per_group = (ws1 - ws0 + kWk - 1) / kWk;
    const int sb0 = min(ws0 + gk * per_group, ws1), sb1 = min(sb0 + per_group, ws1);
    const int sb_end = sb0 + per_group;  // steps run up to here
    const __amdgpu_buffer_rsrc_t rs_w = rsrc(a.wt, (size_t)RB * sb1 * tiled::kChunk);
    const uint32_t chunk_stride = (uint32_t)RB * (uint32_t)tiled::kChunk;
    uint32_t a_off[kAL], w_off[kNT];
#pragma unroll
    for (int q = 0; q < kAL; ++q) a_off[q] = (a_row[q] * (uint32_t)a.K + (uint32_t)spiece * 8u) * 2u;
#pragma unroll
    for (int tn = 0; tn < kNT; ++tn) w_off[tn] = (uint32_t)rb[tn] * (uint32_t)tiled::kChunk + (uint32_t)lane * 16u;
    // half-step hs = 2 sb + g (clamped into the slice) of the activations into stage `stg`: every wave fills the four rows
    // 16 q + 4 wave + [0, 4) of piece q, one contiguous kilobyte of LDS per load
    auto load_x = [&](int hs, int stg) __attribute__((always_inline)) {
      const int h = min(hs, 2 * SB - 1);
      typedef __attribute__((address_space(3))) void* lds_ptr_t;
#pragma unroll
      for (int q = 0; q < kAL; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr_t)(smem + (size_t)stg * BM * kTRow + (16 * q + 4 * wave) * kTRow), 16, (int)a_off[q],
                                                 h * 256, 0, 0);
    };
    // The activations of the next stage have landed before the workgroup's barrier: loads return in order, so it is enough
    // to wait until no more loads are outstanding than were issued behind them (the refills of this half-step, which
    // stay in flight).  The scheduling barriers keep the loads where they are written: left alone, the compiler sinks
    // the refills to the end of the half-step, where nothing hides them.
    auto wait_loads_but = [&](auto n_const) __attribute__((always_inline)) {
      constexpr int n = decltype(n_const)::value;
      __builtin_amdgcn_s_waitcnt((n & 15) | 0x0F70 | ((n >> 4) << 14));  // vmcnt(n), nothing else
    };
    // Two sets of weight registers take turns: while the pieces of one are dequantised, the same pieces of the other are
    // refilled with the next super-block (a set refilled in place would have to be copied at the loop's back edge, and a
    // copy waits for the load).
    struct BSet {
      u32x4 w[kNT][4];
      u32x2 side[kNT];
    };
    BSet b0, b1;
    const int side_off = tiled::kCodeBytes + ln * 8;
    if (ws0 < ws1) {
      load_x(2 * sb0, stage);
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
#pragma unroll
        for (int j = 0; j < 4; ++j) b0.w[tn][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (int)w_off[tn] + j * 1024, sb0 * (int)chunk_stride, 0);
        b0.side[tn] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_w, (int)((uint32_t)rb[tn] * (uint32_t)tiled::kChunk) + side_off,
                                                                                     sb0 * (int)chunk_stride, 0));
      }
      wait_loads_but(std::integral_constant<int, 0>{});
      __syncthreads();
    }
    // g is a compile-time constant at every call site; `cur` holds super-block sb, `nxt` receives sb + 1
    auto half_step = [&](int sb, auto g_const, const BSet& cur, BSet& nxt) __attribute__((always_inline)) {
      constexpr int g = decltype(g_const)::value;
      const int sbn = sb + 1;  // (behind the group's last super-block: past the end of the descriptor, zeros nobody uses)
      if (!(GLOWQ_GDBG & 8)) load_x(2 * sb + g + 1, stage ^ 1);
      if (g == 1) {
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
          nxt.side[tn] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_w, (int)((uint32_t)rb[tn] * (uint32_t)tiled::kChunk) + side_off,
                                                                                        sbn * (int)chunk_stride, 0));
      }
      __builtin_amdgcn_sched_barrier(0);
      h2 zb_lo[kNT], zb_hi[kNT], s2[kNT];
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        const uint32_t sw = cur.side[tn][g];
        const float nz = (float)__builtin_bit_cast(half_t, (uint16_t)(sw >> 16)) * 65536.0f;  // -zero
        const half_t zl = (half_t)(nz - 1024.0f), zh = (half_t)(nz - 64.0f);
        zb_lo[tn] = h2{zl, zl};
        zb_hi[tn] = h2{zh, zh};
        s2[tn] = bitcast_u32<h2>(__builtin_amdgcn_perm(sw, sw, 0x01000100u));
      }
#pragma unroll
      for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
          nxt.w[tn][2 * g + p] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (int)w_off[tn] + (2 * g + p) * 1024, sbn * (int)chunk_stride, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          h8 bf[kNT];
#pragma unroll
          for (int tn = 0; tn < kNT; ++tn)
            bf[tn] = (GLOWQ_GDBG & 1) ? __builtin_bit_cast(h8, u32x4{cur.w[tn][2 * g + p][i], cur.w[tn][2 * g + p][i] ^ cur.side[tn].x, 0u, 0u})
                                      : dequant_word(cur.w[tn][2 * g + p][i], zb_lo[tn], zb_hi[tn], s2[tn]);
#pragma unroll
          for (int c = 0; c < kMT; c += kChunk) {
            h8 af[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; ++u)
              af[u] = (GLOWQ_GDBG & 2) ? __builtin_bit_cast(h8, u32x4{(uint32_t)(c + u + i), (uint32_t)p, (uint32_t)lane, 0u})
                                       : read_a(stage, c + u, 8 * lh + 4 * p + i);
#pragma unroll
            for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
              for (int u = 0; u < kChunk; ++u)
                acc[c + u][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[u], bf[tn], acc[c + u][tn], 0, 0, 0);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      wait_loads_but(std::integral_constant<int, 2 * kNT + (g == 1 ? kNT : 0)>{});
      if (!(GLOWQ_GDBG & 4)) __syncthreads();
      stage ^= 1;
    };
    int sb = sb0;
    for (; sb + 1 < sb_end; sb += 2) {
      half_step(sb, std::integral_constant<int, 0>{}, b0, b1);
      half_step(sb, std::integral_constant<int, 1>{}, b0, b1);
      half_step(sb + 1, std::integral_constant<int, 0>{}, b1, b0);
      half_step(sb + 1, std::integral_constant<int, 1>{}, b1, b0);
    }
    if (sb < sb_end) {
      half_step(sb, std::integral_constant<int, 0>{}, b0, b1);
      half_step(sb, std::integral_constant<int, 1>{}, b0, b1);
    }
  }

  // ---- the second K group hands its accumulators over through LDS (the stages are free: every wave is past the last barrier)
  if constexpr (kWk > 1) {
    float* red = reinterpret_cast<float*>(smem_all);
    if (gk == 1) {
#pragma unroll
      for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
        for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
          for (int i = 0; i < 16; ++i) red[((tm * kNT + tn) * 16 + i) * 256 + tid] = acc[tm][tn][i];
    }
    __syncthreads();
    if (gk == 1) return;
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tm][tn][i] += red[((tm * kNT + tn) * 16 + i) * 256 + tid];
  }

  // ---- epilogue: accumulator register i of a 32x32 tile is row 8*(i/4) + 4*lh + i%4, column ln ---------
  if (nslices > 1) {
    float* part = gg.partials + ((size_t)slice * part_tiles + part_tile) * (BM * BN);
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm)
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
        for (int i = 0; i < 16; ++i) part[((tm * kNT + tn) * 16 + i) * 256 + tid] = acc[tm][tn][i];
    return;
  }
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) {
    const int n = bn * BN + wave * (32 * kNT) + tn * 32 + ln;
    if (n >= a.N) continue;
    const float b = a.bias ? (float)a.bias[n] : 0.f;
#pragma unroll
    for (int tm = 0; tm < kMT; ++tm) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + tm * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < a.M) a.y[(size_t)m * a.ldy + n] = (half_t)(acc[tm][tn][i] + b);
      }
    }
  }
}

// y = fp16(sum over the slices, in slice order, of the partial tiles of gemm_mfma_kernel<kMT, kNT> + bias); same grid
// in x, same workgroup -> (member, row block, column block) map and accumulator-register order as the producer.
// gridDim.y = kMT * kNT: workgroup y of a tile sums one 32 x 32 accumulator tile of each wave (a tile per workgroup
// left the sum of 64 tail tiles to 64 workgroups: 20 us for 34 MB).
template <int kMT, int kNT>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmGroup gg, const int m_blocks) {
  // uniform split: one workgroup per tile of the producer; tail split: one per tail tile (tiles full, full + 1, ...)
  const bool tail = gg.tail_slices > 1;
  const int wg = (tail ? gg.full : 0) + (int)blockIdx.x;
  const int nslices = tail ? gg.tail_slices : gg.slices;
  GemmArgs a = gg.m[0];
  int blk_base = 0;
  for (int i = 1; i < gg.n; ++i)
    if (wg >= gg.blk_end[i - 1]) {
      a = gg.m[i];
      blk_base = gg.blk_end[i - 1];
    }
  constexpr int BM = 32 * kMT, BN = 128 * kNT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ln = lane & 31, lh = lane >> 5;
  const int blk = wg - blk_base;
  const int m0 = (blk % m_blocks) * BM, bn = blk / m_blocks;
  const size_t slice_stride = (size_t)gridDim.x * (BM * BN);
  const float* part = gg.partials + (size_t)blockIdx.x * (BM * BN) + tid;
  const int tn = (int)blockIdx.y % kNT, tm = (int)blockIdx.y / kNT;
  {
    const int n = bn * BN + wave * (32 * kNT) + tn * 32 + ln;
    const float b = (n < a.N && a.bias) ? (float)a.bias[n] : 0.f;
    {
      float v[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = 0.f;
      for (int z = 0; z < nslices; ++z) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] += part[(size_t)z * slice_stride + ((tm * kNT + tn) * 16 + i) * 256];
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + tm * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < a.M && n < a.N) a.y[(size_t)m * a.ldy + n] = (half_t)(v[i] + b);
      }
    }
  }
}

// ---- host side ------------------------------------------------------------------------------------
template <int kMT, int kNT, bool kQuant, bool kSuper = false, bool kTiled = false, int kWk = 1>
static hipError_t launch_gemm_t(GemmGroup& gg, hipStream_t stream) {
  static_assert(!kTiled || (kQuant && kSuper), "the tiled copy serves the super-block form");
  static_assert(kWk == 1 || kTiled, "K groups inside a workgroup: the tiled-copy kernel");
  constexpr int BM = 32 * kMT, BN = 128 * kNT;
  auto kern = kTiled ? gemm_tiled_kernel<kMT, kNT, kWk> : gemm_mfma_kernel<kMT, kNT, kQuant, kSuper>;
  size_t lds = kTiled ? (size_t)kWk * 2 * BM * kTRow
                      : (size_t)2 * BM * kARow * sizeof(half_t) + (kSuper ? (size_t)4 * (32 * kNT) * 144 : 0);
  if (kWk > 1 && lds < (size_t)BM * BN * sizeof(float)) lds = (size_t)BM * BN * sizeof(float);  // the hand-over of the accumulators
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
  note_launch(0, 0, 256 * kWk, "%s<%d,%d,%d>", kTiled ? "gemm_tiled_kernel" : "gemm_mfma_kernel", kMT, kNT, kWk);
  const int m_blocks = (gg.m[0].M + BM - 1) / BM;
  int total = 0;
  for (int i = 0; i < gg.n; ++i) {
    total += m_blocks * ((gg.m[i].N + BN - 1) / BN);
    gg.blk_end[i] = total;
  }
  if (!(kQuant && kSuper)) gg.slices = 1;
  if (!(kQuant && kSuper) || gg.slices > 1 || gg.tail_slices < 2 || gg.full < 0 || gg.full >= total) gg.tail_slices = 0;
  if (gg.tail_slices > 1) {
    const int tail_tiles = total - gg.full;
    hipLaunchKernelGGL(kern, dim3(gg.full + tail_tiles * gg.tail_slices, 1), dim3(256 * kWk), lds, stream, gg, m_blocks);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    hipLaunchKernelGGL((gemm_reduce_kernel<kMT, kNT>), dim3(tail_tiles, kMT * kNT), dim3(256), 0, stream, gg, m_blocks);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(kern, dim3(total, gg.slices), dim3(256 * kWk), lds, stream, gg, m_blocks);
  if (hipError_t e = hipGetLastError(); e != hipSuccess || gg.slices == 1) return e;
  hipLaunchKernelGGL((gemm_reduce_kernel<kMT, kNT>), dim3(total, kMT * kNT), dim3(256), 0, stream, gg, m_blocks);
  return hipGetLastError();
}

static hipError_t launch_gemm_group(GemmGroup& gg, int num_cus, size_t ws_bytes, hipStream_t stream) {
  // Tile choice: the largest tile (most reuse of both operands) whose workgroup count still fills the chip; when
  // none does, the one with the most workgroups.  Row tiles are capped by M (and at 4: 8 spills), column tiles at
  // 2 per wave unless every member is narrow.
  int n_max = 0;
  for (int i = 0; i < gg.n; ++i) n_max = gg.m[i].N > n_max ? gg.m[i].N : n_max;
  const int nt_cap = n_max > 128 ? 2 : 1;
  const int M = gg.m[0].M;
  static const int mt_max = getenv("GLOWQ_GEMM_MT") ? atoi(getenv("GLOWQ_GEMM_MT")) : 4;
  int mt_cap = M > 128 ? 8 : (M > 64 ? 4 : (M > 32 ? 2 : 1));
  if (mt_cap > mt_max) mt_cap = mt_max;
  static const int order[6][2] = {{4, 2}, {2, 2}, {4, 1}, {2, 1}, {1, 2}, {1, 1}};
  int mt = 1, nt = 1;
  long best = -1;
  for (int c = 0; c < 6; ++c) {
    const int cmt = order[c][0], cnt = order[c][1];
    if (cmt > mt_cap || cnt > nt_cap) continue;
    long wgs = 0;
    for (int i = 0; i < gg.n; ++i) wgs += (long)((M + 32 * cmt - 1) / (32 * cmt)) * ((gg.m[i].N + 128 * cnt - 1) / (128 * cnt));
    if (wgs >= num_cus) {
      mt = cmt;
      nt = cnt;
      break;
    }
    if (wgs > best) {
      best = wgs;
      mt = cmt;
      nt = cnt;
    }
  }
  if (mt_cap == 8 && mt == 4 && mt_max >= 8) mt = 8;
  static const int force_mt = getenv("GLOWQ_GEMM_FORCE_MT") ? atoi(getenv("GLOWQ_GEMM_FORCE_MT")) : 0;
  static const int force_nt = getenv("GLOWQ_GEMM_FORCE_NT") ? atoi(getenv("GLOWQ_GEMM_FORCE_NT")) : 0;
  if (force_mt > 0 && force_mt <= mt_cap) mt = force_mt;
  if (force_nt > 0 && force_nt <= nt_cap) nt = force_nt;
  static const int env_super = getenv("GLOWQ_GEMM_SUPER") ? atoi(getenv("GLOWQ_GEMM_SUPER")) : 1;
  // the super-block form addresses its operands with 32-bit byte offsets
  bool fits32 = (size_t)M * gg.m[0].K * 2 < (1ull << 32);
  for (int i = 0; i < gg.n; ++i) {
    const size_t rows = (size_t)gg.m[i].N;
    fits32 = fits32 && rows * gg.m[i].ldw * 4 < (1ull << 32) && rows * gg.m[i].lds * 2 < (1ull << 32) && rows * gg.m[i].ldz * 4 < (1ull << 32);
  }
  const bool super = env_super != 0 && (gg.m[0].K & 255) == 0 && gg.m[0].group_size >= 128 && fits32;
  // the tiled copy of the weights where every member brings one (and its tiled left factor where it is corrected)
  static const int env_tiled = getenv("GLOWQ_GEMM_TILED") ? atoi(getenv("GLOWQ_GEMM_TILED")) : 1;
  bool tiled_ok = super && env_tiled != 0 && tiled::applies(gg.m[0].K, gg.m[0].group_size);
  for (int i = 0; i < gg.n; ++i)
    tiled_ok = tiled_ok && gg.m[i].wt != nullptr && (gg.m[i].r == nullptr || gg.m[i].lt != nullptr) &&
               tiled::weight_bytes(gg.m[i].N, gg.m[i].K) < (1ull << 32);
  // About one 128 x 256 tile per compute unit and a long K (where K would otherwise be cut into slices over workgroups,
  // with fp32 partial tiles through the workspace and a second launch for their sum): eight waves per tile, the K range
  // dealt to two groups of four inside the workgroup (gemm_tiled_kernel's kWk = 2), the sum in LDS.  Qwen2.5-7B down_proj at
  // 2048 rows (K = 18944, 224 tiles): 308 -> 294 us.  On short K it does not pay: o_proj (K = 3584, 224 tiles) 77.5 -> 78.6 us
  // against two co-resident 64 x 256 workgroups per compute unit, q|k|v (288 tiles) 100.6 -> 114.9 (its tail tiles, cut
  // along K, no longer fit beside a whole tile).
  static const int env_wk = getenv("GLOWQ_GEMM_WK") ? atoi(getenv("GLOWQ_GEMM_WK")) : 0;
  int wk = 1;
  if (tiled_ok && mt_cap >= 4 && nt_cap == 2 && env_wk != 1) {
    long tiles42 = 0;
    for (int i = 0; i < gg.n; ++i) tiles42 += (long)((M + 127) / 128) * ((gg.m[i].N + 255) / 256);
    if ((tiles42 * 2 >= num_cus && tiles42 < 2L * num_cus && (gg.m[0].K >> 8) >= 32) || env_wk == 2) {
      mt = 4;
      nt = 2;
      wk = 2;
    }
  }
  // Split K through the workspace: where even the largest tile the rows allow leaves CUs idle, that tile is kept and K
  // is cut into slices of at least sixteen super-blocks until the workgroups number about two per CU.
  static const int env_split = getenv("GLOWQ_GEMM_SPLIT") ? atoi(getenv("GLOWQ_GEMM_SPLIT")) : 1;
  const int ws_slices_fit = gg.slices;  // on entry: how many slices of the whole output the workspace holds
  gg.slices = 1;
  if (super && env_split != 0 && ws_slices_fit >= 2 && mt_cap >= 2 && nt_cap == 2 && wk == 1) {
    const int bmt = mt_cap >= 4 ? 4 : 2;
    long tiles = 0;
    for (int i = 0; i < gg.n; ++i) tiles += (long)((M + 32 * bmt - 1) / (32 * bmt)) * ((gg.m[i].N + 255) / 256);
    const int sb_total = gg.m[0].K >> 8;
    long want = (2L * num_cus) / tiles;
    // every slice writes the whole output once more in fp32, the reduction reads it back, and a short K loop is mostly
    // ramp: only slices of 16 super-blocks and more pay (measured: 2048 x 3584 outputs gain 8 % at K = 18944 in two
    // slices and lose 12 % at K = 3584; 128..512 rows of K = 4096 lose up to 40 % in slices of four super-blocks)
    // ... unless the output has so few tiles that most of the chip would otherwise sit idle for the whole of a long K
    // (4096 outputs of K = 14336 at 65..256 rows: 16 to 32 tiles, 97 -> 75..80 us with slices of four to eight)
    static const int env_depth = getenv("GLOWQ_GEMM_MIN_DEPTH") ? atoi(getenv("GLOWQ_GEMM_MIN_DEPTH")) : 0;
    const long min_depth = env_depth > 0 ? env_depth : (tiles >= 64 ? 16 : (tiles >= 32 ? 8 : 4));
    if (want > sb_total / min_depth) want = sb_total / min_depth;
    if (want > ws_slices_fit) want = ws_slices_fit;
    if (tiles < num_cus && want >= 2 && tiles * want * 2 >= num_cus) {
      mt = bmt;
      nt = 2;
      gg.slices = (int)want;
    }
  }
  // Tail split: the tiles beyond the last multiple of the CU count are cut along K so that the work they add is spread
  // over the whole chip (2368 tiles on 256 CUs: 9.25 tiles' worth of time instead of 10; 288 tiles: 1.125 instead of 2).
  // Only where that tail is at most 0.6 of a round, K leaves every slice two super-blocks or more, and the workspace
  // holds the partial tiles.
  static const int env_tail = getenv("GLOWQ_GEMM_TAIL") ? atoi(getenv("GLOWQ_GEMM_TAIL")) : 1;
  gg.full = 0;
  gg.tail_slices = 0;
  if (super && env_tail != 0 && gg.slices == 1 && ws_bytes > 0) {
    long tiles = 0;
    for (int i = 0; i < gg.n; ++i) tiles += (long)((M + 32 * mt - 1) / (32 * mt)) * ((gg.m[i].N + 128 * nt - 1) / (128 * nt));
    const long tail = tiles % num_cus;
    const int sb_total = gg.m[0].K >> 8;
    // (measured at 2048 rows, projection launch included: 2368 tiles 590 -> 573 us, 288 tiles 119 -> 107 us)
    if (tiles > num_cus && tail > 0 && tail * 10 <= (long)num_cus * 6) {
      long s_want = num_cus / tail;
      if (s_want > 8) s_want = 8;
      if (s_want > sb_total / 2) s_want = sb_total / 2;
      const size_t tile_bytes = (size_t)(32 * mt) * (128 * nt) * sizeof(float);
      while (s_want >= 2 && (size_t)tail * s_want * tile_bytes > ws_bytes) --s_want;
      if (s_want >= 2) {
        // (slices of equal depth: no more of them than leave none empty)
        const int per = (sb_total + (int)s_want - 1) / (int)s_want;
        gg.tail_slices = (sb_total + per - 1) / per;
        gg.full = (int)(tiles - tail);
      }
    }
  }
  if (wk == 2) return launch_gemm_t<4, 2, true, true, true, 2>(gg, stream);
#define GLOWQ_GEMM_CASE(MT, NT)                                                            \
  if (mt == MT && nt == NT)                                                                \
    return tiled_ok ? launch_gemm_t<MT, NT, true, true, true>(gg, stream)                  \
           : super  ? launch_gemm_t<MT, NT, true, true>(gg, stream)                        \
                    : launch_gemm_t<MT, NT, true>(gg, stream);
  GLOWQ_GEMM_CASE(8, 2) GLOWQ_GEMM_CASE(4, 2) GLOWQ_GEMM_CASE(2, 2) GLOWQ_GEMM_CASE(1, 2)
  GLOWQ_GEMM_CASE(8, 1) GLOWQ_GEMM_CASE(4, 1) GLOWQ_GEMM_CASE(2, 1) GLOWQ_GEMM_CASE(1, 1)
#undef GLOWQ_GEMM_CASE
  return hipErrorInvalidValue;
}

// The MFMA route needs 64-deep k blocks that stay inside one quantisation group per 32-column half and
// 16-byte aligned rows everywhere.
bool gemm_supported(const GroupDev& g) {
  if ((g.K % kBK) != 0 || (g.group_size % 32) != 0 || (g.group_size & (g.group_size - 1)) != 0) return false;
  // r is either given or still to be produced from R into r_out by the projection launch that goes ahead
  const half_t* r = g.r != nullptr ? g.r : (g.R != nullptr ? g.r_out : nullptr);
  if (r != nullptr && ((g.rank & 7) != 0 || g.rank < 8)) return false;
  if ((reinterpret_cast<uintptr_t>(g.x) & 15u) != 0) return false;
  if (r != nullptr && (reinterpret_cast<uintptr_t>(r) & 15u) != 0) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if ((reinterpret_cast<uintptr_t>(m.qweight) & 15u) != 0 || (m.ldw & 3) != 0) return false;
    if (m.L != nullptr && (reinterpret_cast<uintptr_t>(m.L) & 15u) != 0) return false;
  }
  return true;
}

hipError_t launch_gemm(GroupDev& g, int num_cus, hipStream_t stream) {
  GemmGroup gg;
  gg.n = g.n_members;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    GemmArgs& a = gg.m[i];
    a.x = g.x;
    a.r = (m.L != nullptr) ? g.r : nullptr;
    a.qweight = m.qweight;
    a.scales = m.scales;
    a.qzeros = m.qzeros;
    a.bmat = m.L;
    a.bias = m.bias;
    a.y = m.y;
    a.wt = static_cast<const unsigned char*>(m.tiled);
    a.lt = (m.L != nullptr && m.tiled_L != nullptr && m.tiled_rank == g.rank) ? static_cast<const unsigned char*>(m.tiled_L) : nullptr;
    a.M = g.M;
    a.N = m.N;
    a.K = g.K;
    a.group_size = g.group_size;
    a.rank = g.rank;
    a.ldw = m.ldw;
    a.lds = m.lds;
    a.ldz = m.ldz;
    a.ldb = g.rank;
    a.ldy = m.ldy;
    a.alpha = g.alpha;
  }
  // slices of the padded output (rows to a multiple of 128, columns of every member to a multiple of 256) that fit the
  // workspace; launch_gemm_group turns this into the slice count
  size_t padded = 0;
  for (int i = 0; i < g.n_members; ++i) padded += (size_t)((g.M + 127) / 128 * 128) * ((g.mem[i].N + 255) / 256 * 256);
  const bool ws_ok = g.ws != nullptr && (reinterpret_cast<uintptr_t>(g.ws) & 15u) == 0;
  gg.slices = ws_ok ? (int)std::min<size_t>(g.ws_bytes / (padded * sizeof(float)), 64) : 0;
  gg.partials = static_cast<float*>(g.ws);
  return launch_gemm_group(gg, num_cus, ws_ok ? g.ws_bytes : 0, stream);
}

// ---- shared projection for many rows: r[M, rank] = fp16(x[M, K] . R[rank, K]^T) ---------------------------
// N = rank is tiny, so the parallelism has to come from M and K: a workgroup owns 32 rows of x and up to 128
// columns of r, and its four waves split K -- wave w takes the 64-deep slice w of every 256-deep block, with
// its own A fragments (x, staged in LDS for all four slices at once) and its own B fragments (R, straight
// from global memory, prefetched one block ahead).  There is no barrier-bound dependency between the waves
// inside a block beyond the staging of x; the four partial tiles meet in LDS once, at the end.
constexpr int kPK = 256;           // k depth of one block (4 waves x 64)
constexpr int kPRow = kPK + 8;     // padded LDS row in halves

//
// Split K (gridDim.z > 1): workgroup z of a tile takes a contiguous range of blocks and leaves its fp32 partial tile
// in the caller's workspace, [tile][slice][kNT * 1024] floats in accumulator-register order; proj_reduce_kernel then
// adds the partials in slice order and writes r.  (Finishing a tile in the workgroup that arrives last at a counter
// was measured first: the device-scope traffic it needs inside one launch costs 20 us and more, a second launch 4.)
struct ProjSplit {
  float* partials;
};

template <int kNT>
__global__ __launch_bounds__(256) void proj_mfma_kernel(const half_t* __restrict__ x, const half_t* __restrict__ R,
                                                        half_t* __restrict__ r, int M, int K, int rank, ProjSplit sp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  half_t* lds_x = reinterpret_cast<half_t*>(smem);  // [2][32][kPRow]; reused for the final reduction
  constexpr size_t kLdsX = (size_t)2 * 32 * kPRow * sizeof(half_t), kLdsRed = (size_t)4 * kNT * 16 * 64 * 4;
  constexpr size_t b_tile_offset = kLdsX > kLdsRed ? kLdsX : kLdsRed;  // the waves' B tiles lie behind both
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int ln = lane & 31, lh = lane >> 5;
  const int m0 = blockIdx.x * 32;
  const int n0 = blockIdx.y * (32 * kNT);
  const int all_blocks = (K + kPK - 1) / kPK;  // K is a multiple of 64; the last block may be partial
  const int slices = gridDim.z;
  const int per_slice = (all_blocks + slices - 1) / slices;
  const int blk_begin = min((int)blockIdx.z * per_slice, all_blocks);
  const int blocks = min(blk_begin + per_slice, all_blocks);  // this workgroup walks blocks [blk_begin, blocks)

  f16v acc[kNT];
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[tn][i] = 0.f;

  // x tile of a block: 32 rows x 32 octets; thread t takes octets t, t+256, t+512, t+768
  struct XRegs {
    u32x4 v[4];
  };
  auto load_x = [&](int kb, XRegs& xr) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = tid + 256 * i;
      const int row = min(m0 + (q >> 5), M - 1);
      const int k = min(kb + (q & 31) * 8, K - 8);
      xr.v[i] = *reinterpret_cast<const u32x4*>(x + (size_t)row * K + k);
    }
  };
  auto store_x = [&](int stage, const XRegs& xr) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = tid + 256 * i;
      *reinterpret_cast<u32x4*>(lds_x + ((size_t)stage * 32 + (q >> 5)) * kPRow + (q & 31) * 8) = xr.v[i];
    }
  };
  // R reaches the B operand through a wave-private LDS tile: the wave's 128-byte row segments (its 64-column slice of
  // 32 kNT rows of R) are loaded in memory order, 8 lanes per segment, and read back in MFMA lane order.  Fragment
  // loads straight from memory put every lane of a request on a line of its own.
  constexpr int kSeg = 144;  // bytes per row segment in the tile: 128 + 16, conflict-free fragment reads
  unsigned char* btile = smem + b_tile_offset + (size_t)wave * (32 * kNT) * kSeg;
  struct BRegs {
    u32x4 w[kNT * 4];  // row 8 q + lane / 8 of the tile, piece lane % 8
  };
  // this wave's slice of a block: columns kb + 64*wave .. +63; a slice past the end of K is weighted by zero
  auto load_b = [&](int kb, BRegs& br) {
    const int ks = min(kb + 64 * wave, K - 64);
#pragma unroll
    for (int q = 0; q < kNT * 4; ++q)
      br.w[q] = *reinterpret_cast<const u32x4*>(R + (size_t)min(n0 + q * 8 + (lane >> 3), rank - 1) * K + ks + (lane & 7) * 8);
  };
  auto stage_b = [&](const BRegs& br) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // fragment reads of the previous block are done
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < kNT * 4; ++q)
      *reinterpret_cast<u32x4*>(btile + (q * 8 + (lane >> 3)) * kSeg + (lane & 7) * 16) = br.w[q];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  auto mma_block = [&](int stage, int kb) {
    if (kb + 64 * wave >= K) return;  // wave-uniform: nothing of this slice lies inside K
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const h8 af = *reinterpret_cast<const h8*>(lds_x + ((size_t)stage * 32 + ln) * kPRow + 64 * wave + (4 * lh + t) * 8);
#pragma unroll
      for (int tn = 0; tn < kNT; ++tn) {
        const h8 bf = *reinterpret_cast<const h8*>(btile + (tn * 32 + ln) * kSeg + lh * 64 + t * 16);
        acc[tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[tn], 0, 0, 0);
      }
    }
  };

  int stage = 0;
  // Block s: move B(s) out of its register set into the wave's LDS tile, refill that set with B(s+2) and the matching x set with
  // x(s+2), run the MFMAs of block s on LDS stage s%2, then move x(s+1) (loaded one block ago) into the other
  // stage.  Two blocks of loads are in flight at any time.
  auto block = [&](int blk, BRegs& br, XRegs& x_fill, const XRegs& x_store) {
    stage_b(br);
    const int kn = min(blk + 2, all_blocks - 1) * kPK;
    load_b(kn, br);
    load_x(kn, x_fill);
    mma_block(stage, blk * kPK);
    store_x(stage ^ 1, x_store);
    __syncthreads();
    stage ^= 1;
  };
  XRegs x0, x1;
  BRegs b0, b1;
  load_x(min(blk_begin, all_blocks - 1) * kPK, x0);
  load_b(min(blk_begin, all_blocks - 1) * kPK, b0);
  load_x(min(blk_begin + 1, all_blocks - 1) * kPK, x1);
  load_b(min(blk_begin + 1, all_blocks - 1) * kPK, b1);
  store_x(0, x0);
  __syncthreads();
  for (int blk = blk_begin; blk < blocks; blk += 2) {
    block(blk, b0, x0, x1);
    if (blk + 1 >= blocks) break;
    block(blk + 1, b1, x1, x0);
  }

  // the four K slices meet in LDS: [wave][tile][16 regs][64 lanes] floats
  float* red = reinterpret_cast<float*>(smem);
  __syncthreads();
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn)
#pragma unroll
    for (int i = 0; i < 16; ++i) red[((wave * kNT + tn) * 16 + i) * 64 + lane] = acc[tn][i];
  __syncthreads();
  // wave w finishes registers 4w .. 4w+3 of every tile
#pragma unroll
  for (int tn = 0; tn < kNT; ++tn) {
    const int n = n0 + tn * 32 + ln;
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int i = wave * 4 + ii;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) v += red[((w * kNT + tn) * 16 + i) * 64 + lane];
      if (slices == 1) {
        const int m = m0 + 8 * (i >> 2) + 4 * lh + (i & 3);
        if (m < M && n < rank) r[(size_t)m * rank + n] = (half_t)v;
      } else {
        const size_t tile = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
        sp.partials[(tile * slices + blockIdx.z) * (kNT * 1024) + (tn * 16 + i) * 64 + lane] = v;
      }
    }
  }
}

// r[m, n] = fp16(sum over the slices, in slice order, of the partial tiles of proj_mfma_kernel<kNT>).  One thread per
// accumulator element of a tile; m_blocks = gridDim.x of the producing launch.
__global__ __launch_bounds__(256) void proj_reduce_kernel(const float* __restrict__ partials, half_t* __restrict__ r, int M,
                                                          int rank, int nt, int slices, int m_blocks) {
  const int per_tile = nt * 1024;
  const int e = blockIdx.x * blockDim.x + threadIdx.x;  // element of the tile: (tn * 16 + i) * 64 + lane
  const int tile = blockIdx.y;
  if (e >= per_tile) return;
  const int lane = e & 63, i = (e >> 6) & 15, tn = e >> 10;
  const int m = (tile % m_blocks) * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
  const int n = (tile / m_blocks) * (32 * nt) + tn * 32 + (lane & 31);
  const float* src = partials + (size_t)tile * slices * per_tile + e;
  float v = 0.f;
  int z = 0;
  for (; z + 8 <= slices; z += 8) {
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) t[u] = src[(size_t)(z + u) * per_tile];
#pragma unroll
    for (int u = 0; u < 8; ++u) v += t[u];
  }
  for (; z < slices; ++z) v += src[(size_t)z * per_tile];
  if (m < M && n < rank) r[(size_t)m * rank + n] = (half_t)v;
}

// How a projection is cut: columns per workgroup (32 * nt) and K slices.  The tile width follows the workgroup count
// (narrow tiles where 64 columns each would leave CUs idle; R is small, re-reading it is cheap).  K is split only with a
// workspace, where the tiles alone fill less than half the chip and K is long enough for the second launch to pay
// (from 4096 columns): then as many slices as bring the workgroup count to about two per CU, each at least two
// blocks deep, as far as the workspace reaches.
struct ProjPlan {
  int nt, slices;
};
static ProjPlan plan_proj(int M, int K, int rank, int num_cus, size_t ws_bytes) {
  const int m_blocks = (M + 31) / 32;
  const int blocks = (K + kPK - 1) / kPK;
  ProjPlan best;
  best.slices = 1;
  best.nt = (m_blocks * ((rank + 63) / 64) < num_cus && rank > 32) ? 1 : 2;
  if (blocks < 16) return best;
  long best_wgs = (long)m_blocks * ((rank + 32 * best.nt - 1) / (32 * best.nt));
  // with a workspace: the tile width whose split brings the most workgroups (up to two per CU); the wider tile on a
  // tie, since x is then read fewer times
  for (int nt : {2, 1}) {
    if (nt == 2 && rank <= 32) continue;
    const long tiles = (long)m_blocks * ((rank + 32 * nt - 1) / (32 * nt));
    if (tiles * 2 > num_cus || tiles > 65535) continue;
    long want = (2L * num_cus + tiles - 1) / tiles;
    const int min_depth = tiles >= 16 ? 4 : 2;  // blocks per slice: the partials of many tiles are traffic of their own
    if (want > blocks / min_depth) want = blocks / min_depth;
    const long fit = (long)(ws_bytes / sizeof(float) / ((size_t)tiles * nt * 1024));
    if (want > fit) want = fit;
    if (want < 2) continue;
    long wgs = tiles * want;
    if (wgs > 2L * num_cus) wgs = 2L * num_cus;
    if (wgs > best_wgs) {
      best_wgs = wgs;
      best.nt = nt;
      best.slices = (int)want;
    }
  }
  return best;
}

size_t proj_workspace_bytes(int M, int K, int rank, int num_cus) {
  if (M <= 16 || (K % kBK) != 0) return 0;
  const ProjPlan p = plan_proj(M, K, rank, num_cus, ~(size_t)0 >> 8);
  if (p.slices < 2) return 0;
  const long tiles = (long)((M + 31) / 32) * ((rank + 32 * p.nt - 1) / (32 * p.nt));
  return (size_t)tiles * p.slices * p.nt * 1024 * sizeof(float);
}

template <int NT>
static hipError_t launch_proj_t(const half_t* x, const half_t* R, half_t* r, int M, int K, int rank, int slices, void* ws,
                                hipStream_t stream) {
  const int m_blocks = (M + 31) / 32;
  const size_t lds_x = (size_t)2 * 32 * kPRow * sizeof(half_t);
  const size_t lds_red = (size_t)4 * NT * 16 * 64 * 4;
  const size_t lds = (lds_x > lds_red ? lds_x : lds_red) + (size_t)4 * (32 * NT) * 144;  // + the four waves' B tiles
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(proj_mfma_kernel<NT>), lds, lds_limit); e != hipSuccess) return e;
  ProjSplit sp = {slices > 1 ? static_cast<float*>(ws) : nullptr};
  const int col_blocks = (rank + 32 * NT - 1) / (32 * NT);
  hipLaunchKernelGGL(proj_mfma_kernel<NT>, dim3(m_blocks, col_blocks, slices), dim3(256), lds, stream, x, R, r, M, K, rank, sp);
  if (hipError_t e = hipGetLastError(); e != hipSuccess || slices == 1) return e;
  hipLaunchKernelGGL(proj_reduce_kernel, dim3(NT * 4, m_blocks * col_blocks), dim3(256), 0, stream, sp.partials, r, M, rank, NT,
                     slices, m_blocks);
  return hipGetLastError();
}

hipError_t launch_shared_proj_mfma(const half_t* x, const half_t* R, half_t* r, int M, int K, int rank, int num_cus,
                                   hipStream_t stream, void* ws, size_t ws_bytes) {
  if ((K % kBK) != 0 || K < kBK) return hipErrorInvalidValue;
  if (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 15u) != 0) ws_bytes = 0;
  const ProjPlan p = plan_proj(M, K, rank, num_cus, ws_bytes);
  if (p.nt == 2) return launch_proj_t<2>(x, R, r, M, K, rank, p.slices, ws, stream);
  return launch_proj_t<1>(x, R, r, M, K, rank, p.slices, ws, stream);
}

}  // namespace glowq
