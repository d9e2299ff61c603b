// Decode GEMV for one to four token rows on gfx950 with every request of a wave in flight before anything is consumed:
// the plain group launch of the kernel in stream_kernel.hpp (what it does and why is described there).
#include <atomic>
#include <cstdlib>

#include "stream_kernel.hpp"

namespace glowq {

using namespace streamk;

// gemv.hip: LDS layout of the staged activations, shared by both single-row kernels
size_t wave_dot_lds_bytes(int M, int K, int rank, bool has_r);

// ---- host side ---------------------------------------------------------------------------------------------
// The stream GEMV takes up to four token rows on the fast layout with quantisation groups of 128 columns and more (a
// pair of steps then holds at most 32 groups of a row: one per lane of a half wave), K up to 9 steps of 2048 columns,
// ranks up to 256, and activations that the workgroup can fetch in four (eight) requests per thread and token row.
bool stream_supported(const GroupDev& g) {
  if (g.M < 1 || g.M > 4 || (g.K & 31) != 0 || g.K > 9 * 2048) return false;
  if (g.group_size < 128 || (g.group_size & (g.group_size - 1)) != 0) return false;
  // r is either given or still to be produced from R into r_out by the projection launch that goes ahead of the group
  const half_t* r = g.r != nullptr ? g.r : (g.R != nullptr ? g.r_out : nullptr);
  const bool has_r = r != nullptr;
  if (has_r && ((g.rank & 1) != 0 || g.rank > 256 || g.rank < 2 || (reinterpret_cast<uintptr_t>(r) & 3u) != 0)) return false;
  if ((reinterpret_cast<uintptr_t>(g.x) & 15u) != 0) return false;
  for (int i = 0; i < g.n_members; ++i) {
    const MemberDev& m = g.mem[i];
    if ((reinterpret_cast<uintptr_t>(m.qweight) & 15u) != 0 || (m.ldw & 3) != 0) return false;
    if (m.L && (reinterpret_cast<uintptr_t>(m.L) & 3u) != 0) return false;
    // 32-bit byte offsets inside every buffer of a member
    if ((long)m.N * m.ldw * 4 >= (1L << 31)) return false;
  }
  return wave_dot_lds_bytes(g.M, g.K, g.rank, has_r) <= 160 * 1024;
}

namespace {

int env_int_s(const char* name, int fallback) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

// kPro: kProPlain, or kProProj where run_group left the projection to the launch (g.pub set, g.R still there)
template <int kKit, int kLW, int kM, bool kPacked, int kPro = kProPlain>
hipError_t launch_stream_p(GroupDev& g, int waves, hipStream_t stream) {
  {
    auto kern = gemv_stream_kernel<kKit, kLW, kM, kPacked, kPro, kEpiNone, stream_xw(kKit), 0>;
    constexpr bool kProj = kPro == kProProj;
    const size_t lds = wave_dot_lds_bytes(kM, g.K, g.rank, g.r != nullptr || kProj);
    static LdsLimit lds_limit;
    if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
    int total = 0, grid = 0;
    for (int i = 0; i < g.n_members; ++i) {
      const int blocks = (g.mem[i].N + kSRows - 1) / kSRows;
      total += blocks;
      g.task_end[i] = total;
      grid += (blocks + waves - 1) / waves;
      g.wg_end[i] = grid;
    }
    ChainDev ch{};
    if constexpr (kProj) {
      grid = front_grid(grid, proj_front_wgs(g.K >> 3, waves, g.rank));  // with the workgroups that produce r, and the collector's
      // Only where every workgroup of the launch is on the chip at once.  A workgroup that is done before r is there
      // waits for it; where a later workgroup waits for its place, that wait costs the launch what the projection
      // launch in front would have, and the workgroups in front take places of their own (the gate|up launch of an 8B
      // layer, 7 workgroups per compute unit: 16.1 to 16.6 us against 15.9 to 16.5; the down_proj launch of a 14B
      // layer, one workgroup per compute unit and two rounds as it is: 23.9 against 19.8).
      // (asked once per instantiation, workgroup size and LDS size; the last answer is kept)
      static std::atomic<long> asked_for{-1};
      static std::atomic<int> resident{0};
      const long shape = (long)lds * 4096 + waves * kWave;
      int per_cu = 0;
      if (asked_for.load(std::memory_order_acquire) == shape) {
        per_cu = resident.load(std::memory_order_relaxed);
      } else {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), waves * kWave, lds) != hipSuccess) per_cu = 0;
        resident.store(per_cu, std::memory_order_relaxed);
        asked_for.store(shape, std::memory_order_release);
      }
      static const int force = env_int_s("GLOWQ_PROJ_FORCE", 0);  // (for measurements: the form on every grid)
      if (!force && !g.pub_mute && (long)grid > (long)per_cu * num_cus()) return hipErrorNotReady;  // the caller launches the projection
      ch.proj_R = g.R;
      ch.proj_r_out = g.r_out;
      ch.proj_pub = g.pub;
      ch.proj_spin = g.pub_spin;
            ch.proj_mute = g.pub_mute;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * kWave), lds, stream, g.x, kProj ? nullptr : g.r, g.K,
                       (g.r || kProj) ? g.rank : 0, g.group_size, g.alpha, g, ch);
    note_launch(grid, 1, waves * kWave, "gemv_stream_kernel<%d,%d,%d,%d,%d,%d,%d,%d>", kKit, kLW, kM, (int)kPacked, kPro, kEpiNone,
                stream_xw(kKit), 0);
    return hipGetLastError();
  }
}

template <int kKit, int kLW>
hipError_t launch_stream_m(GroupDev& g, int waves, hipStream_t stream) {
  bool packed = true;
  for (int i = 0; i < g.n_members; ++i) packed = packed && g.mem[i].side != nullptr;
  switch (g.M) {
    case 1:
      if constexpr (kLW > 0) {
        if (g.pub != nullptr)
          return packed ? launch_stream_p<kKit, kLW, 1, true, kProProj>(g, waves, stream)
                        : launch_stream_p<kKit, kLW, 1, false, kProProj>(g, waves, stream);
      }
      return packed ? launch_stream_p<kKit, kLW, 1, true>(g, waves, stream) : launch_stream_p<kKit, kLW, 1, false>(g, waves, stream);
    case 2: return launch_stream_p<kKit, kLW, 2, false>(g, waves, stream);  // side streams serve single rows only
    case 3: return launch_stream_p<kKit, kLW, 3, false>(g, waves, stream);
    case 4: return launch_stream_p<kKit, kLW, 4, false>(g, waves, stream);
    default: return hipErrorInvalidValue;
  }
}

template <int kKit>
hipError_t launch_stream_lw(GroupDev& g, int waves, hipStream_t stream) {
  const int lw = (g.r || g.pub) ? (g.rank + 127) / 128 : 0;
  if (lw == 0) return launch_stream_m<kKit, 0>(g, waves, stream);
  if (lw == 1) return launch_stream_m<kKit, 1>(g, waves, stream);
  if (lw == 2) return launch_stream_m<kKit, 2>(g, waves, stream);
  return hipErrorInvalidValue;  // ranks above 256 belong to the wave-dot GEMV (stream_supported)
}

}  // namespace

hipError_t launch_stream(GroupDev& g, int num_cus, hipStream_t stream) {
  (void)num_cus;
  const int U = g.K >> 5;
  const int kit = (U + kWave - 1) / kWave;
  long blocks = 0;
  for (int i = 0; i < g.n_members; ++i) blocks += (g.mem[i].N + kSRows - 1) / kSRows;
  // 4 waves per workgroup, 8 for the long groups (measured: q|k|v 5.1 us at 4 against 5.6 at 8, down_proj 8.7 against 9.5,
  // gate|up 13.5 against 13.3)
  static const int env_waves = env_int_s("GLOWQ_STREAM_WAVES", 0);
  // (with more than one token row the long-K instantiations want 8 as well: down_proj at three rows 13.4 us against 18.2)
  int waves = env_waves > 0 ? env_waves : ((blocks >= 8192 || (g.M > 1 && stream_heavy(kit))) ? 8 : 4);
  const int max_waves = stream_heavy(kit) ? 8 : 16;
  if (waves > max_waves) waves = max_waves;
  while ((g.K >> 3) > stream_xw(kit) * waves * kWave && waves < max_waves) ++waves;
  if ((g.K >> 3) > stream_xw(kit) * waves * kWave) return hipErrorInvalidValue;
  switch (kit) {
    case 1: return launch_stream_lw<1>(g, waves, stream);
    case 2: return launch_stream_lw<2>(g, waves, stream);
    case 3: return launch_stream_lw<3>(g, waves, stream);
    case 4: return launch_stream_lw<4>(g, waves, stream);
    case 5: return launch_stream_lw<5>(g, waves, stream);
    case 6: return launch_stream_lw<6>(g, waves, stream);
    case 7: return launch_stream_lw<7>(g, waves, stream);
    case 8: return launch_stream_lw<8>(g, waves, stream);
    case 9: return launch_stream_lw<9>(g, waves, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace glowq
