// The chained single-token forms of the stream GEMV (stream_kernel.hpp): a group launch that applies the RMSNorm in
// front of it while staging its activations and takes its correction's r from an accumulator, and/or ends in the
// residual add or the SwiGLU gate behind it and adds its rows' share of the next group's projection to an accumulator.
#include <cstdlib>

#include "stream_kernel.hpp"

namespace glowq {

using namespace streamk;

size_t wave_dot_lds_bytes(int M, int K, int rank, bool has_r);  // gemv.hip
bool stream_supported(const GroupDev& g);                       // gemv_stream.hip

namespace {

template <int kKit, int kLW, int kPro, int kEpi, bool kW8>
hipError_t launch_chain_w(GroupDev& g, ChainDev ch, int waves, hipStream_t stream) {
  auto kern = gemv_stream_kernel<kKit, kLW, 1, false, kPro, kEpi, chain_xw(kKit, kW8), chain_acc_loads(kW8)>;
  const size_t lds = wave_dot_lds_bytes(1, g.K, g.rank, true) + chain_extra_lds(waves, g.rank);
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), lds, lds_limit); e != hipSuccess) return e;
  int total = 0, grid = 0;
  for (int i = 0; i < (kEpi == kEpiSwiglu ? 1 : g.n_members); ++i) {
    // a gate/up pair: one row of each member per wave; otherwise two rows of a member
    const int blocks = kEpi == kEpiSwiglu ? g.mem[i].N : (g.mem[i].N + kSRows - 1) / kSRows;
    total += blocks;
    g.task_end[i] = total;
    grid += (blocks + waves - 1) / waves;
    g.wg_end[i] = grid;
  }
  ch.part_limit = 0x1p31f / (float)grid;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * kWave), lds, stream, g.x, kPro == kProPlain ? g.r : nullptr, g.K, g.rank,
                     g.group_size, g.alpha, g, ch);
  return hipGetLastError();
}

template <int kKit, int kLW, int kPro, int kEpi>
hipError_t launch_chain_i(GroupDev& g, const ChainDev& ch, int waves, hipStream_t stream) {
  return waves >= 8 ? launch_chain_w<kKit, kLW, kPro, kEpi, true>(g, ch, waves, stream)
                    : launch_chain_w<kKit, kLW, kPro, kEpi, false>(g, ch, waves, stream);
}

template <int kKit, int kLW>
hipError_t launch_chain_pe(GroupDev& g, const ChainDev& ch, int pro, int epi, int waves, hipStream_t stream) {
  // the combinations a decoder layer uses: q|k|v, o_proj, gate|up (behind a norm of its own or a norm launch), down_proj
  if (pro == kProNormAcc && epi == kEpiNone) return launch_chain_i<kKit, kLW, kProNormAcc, kEpiNone>(g, ch, waves, stream);
  if (pro == kProPlain && epi == kEpiResidual) return launch_chain_i<kKit, kLW, kProPlain, kEpiResidual>(g, ch, waves, stream);
  if (pro == kProNormAcc && epi == kEpiSwiglu) return launch_chain_i<kKit, kLW, kProNormAcc, kEpiSwiglu>(g, ch, waves, stream);
  if (pro == kProAcc && epi == kEpiResidual) return launch_chain_i<kKit, kLW, kProAcc, kEpiResidual>(g, ch, waves, stream);
  if (pro == kProPlain && epi == kEpiSwiglu) return launch_chain_i<kKit, kLW, kProPlain, kEpiSwiglu>(g, ch, waves, stream);
  return hipErrorInvalidValue;
}

template <int kKit>
hipError_t launch_chain_lw(GroupDev& g, const ChainDev& ch, int pro, int epi, int waves, hipStream_t stream) {
  return g.rank <= 128 ? launch_chain_pe<kKit, 1>(g, ch, pro, epi, waves, stream)
                       : launch_chain_pe<kKit, 2>(g, ch, pro, epi, waves, stream);
}

}  // namespace

// The combinations served: (norm + accumulator, none), (plain, residual), (norm + accumulator, SwiGLU),
// (plain, SwiGLU), (accumulator, residual).
bool chain_combination_supported(int pro, int epi) {
  return (pro == kProNormAcc && (epi == kEpiNone || epi == kEpiSwiglu)) || (epi == kEpiResidual && (pro == kProPlain || pro == kProAcc)) ||
         (pro == kProPlain && epi == kEpiSwiglu);
}

hipError_t launch_stream_chained(GroupDev& g, const ChainDev& ch, int pro, int epi, hipStream_t stream) {
  const int U = g.K >> 5;
  const int kit = (U + kWave - 1) / kWave;
  long blocks = 0;
  for (int i = 0; i < g.n_members; ++i) blocks += (g.mem[i].N + kSRows - 1) / kSRows;
  // waves per workgroup as in the plain launch (GLOWQ_CHAIN_WAVES overrides, for tuning runs)
  static const int env_waves = getenv("GLOWQ_CHAIN_WAVES") ? atoi(getenv("GLOWQ_CHAIN_WAVES")) : 0;
  static const int env_heavy = getenv("GLOWQ_CHAIN_WAVES_HEAVY") ? atoi(getenv("GLOWQ_CHAIN_WAVES_HEAVY")) : 0;
  int waves = stream_heavy(kit) ? (env_heavy >= 4 ? env_heavy : 8) : (env_waves >= 4 ? env_waves : (blocks >= 8192 ? 8 : 4));
  const int max_waves = stream_heavy(kit) ? 8 : 16;
  if (waves > max_waves) waves = max_waves;
  while ((g.K >> 3) > chain_xw(kit, waves >= 8) * waves * kWave && waves < max_waves) ++waves;
  if ((g.K >> 3) > chain_xw(kit, waves >= 8) * waves * kWave) return hipErrorInvalidValue;
  switch (kit) {
    case 1: return launch_chain_lw<1>(g, ch, pro, epi, waves, stream);
    case 2: return launch_chain_lw<2>(g, ch, pro, epi, waves, stream);
    case 3: return launch_chain_lw<3>(g, ch, pro, epi, waves, stream);
    case 4: return launch_chain_lw<4>(g, ch, pro, epi, waves, stream);
    case 5: return launch_chain_lw<5>(g, ch, pro, epi, waves, stream);
    case 6: return launch_chain_lw<6>(g, ch, pro, epi, waves, stream);
    case 7: return launch_chain_lw<7>(g, ch, pro, epi, waves, stream);
    case 8: return launch_chain_lw<8>(g, ch, pro, epi, waves, stream);
    case 9: return launch_chain_lw<9>(g, ch, pro, epi, waves, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace glowq
