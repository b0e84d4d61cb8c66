#include "common.h"
namespace axl {
size_t flash_bwd_workspace_bytes(const AxlFlashBwdParams& p) { return 16; }
int launch_flash_bwd(const AxlFlashBwdParams& p, hipStream_t stream) {
  return set_error(AXL_ERR_UNSUPPORTED, "axl_flash_bwd: not built yet");
}
}  // namespace axl
