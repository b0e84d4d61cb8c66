#include "common.h"
namespace axl {
size_t paged_decode_workspace_bytes(const AxlPagedDecodeParams& p) { return 16; }
int launch_paged_decode(const AxlPagedDecodeParams& p, hipStream_t stream) {
  return set_error(AXL_ERR_UNSUPPORTED, "axl_paged_decode: not built yet");
}
size_t decode_workspace_bytes(const AxlDecodeParams& p) { return 16; }
int launch_decode(const AxlDecodeParams& p, hipStream_t stream) {
  return set_error(AXL_ERR_UNSUPPORTED, "axl_decode: not built yet");
}
}  // namespace axl
