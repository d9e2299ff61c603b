// placeholder: skinny MFMA route not built yet
#include "common.hpp"
namespace glowq {
bool skinny_supported(const GroupDev&) { return false; }
hipError_t launch_skinny(GroupDev&, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace glowq
