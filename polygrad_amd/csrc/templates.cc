// Hand-written kernel templates selected by pattern match on the scheduled
// root: MFMA matmul and the guarded embedding gather.
#include "render_hip.h"

namespace polyhip {

bool try_render_matmul(const KernelGraph &, const std::string &, const RenderOptions &, RenderedKernel *) {
  return false;
}
bool try_render_gather(const KernelGraph &, const std::string &, const RenderOptions &, RenderedKernel *) {
  return false;
}

}  // namespace polyhip
