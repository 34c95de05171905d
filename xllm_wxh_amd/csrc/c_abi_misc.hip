// Status plumbing of the C ABI.
#include "host_utils.h"

namespace xllm_hip {
char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace xllm_hip

extern "C" const char* xllm_hip_last_error(void) { return xllm_hip::last_error_buffer(); }

extern "C" int xllm_hip_abi_version(void) { return XLLM_HIP_ABI_VERSION; }
