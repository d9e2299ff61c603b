// placeholder: tiled MFMA GEMM route not built yet
#include "common.hpp"
namespace glowq {
bool gemm_supported(const GroupDev&) { return false; }
hipError_t launch_gemm(GroupDev&, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_shared_proj_mfma(const half_t*, const half_t*, half_t*, int, int, int, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace glowq
