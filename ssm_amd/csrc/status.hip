// Status strings and the per-thread error detail of the C ABI.
#include "common.hpp"

#include <string.h>

namespace ssm {

static thread_local char g_last_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

}  // namespace ssm

extern "C" int ssm_amd_abi_version(void) { return SSM_AMD_ABI_VERSION; }

extern "C" const char *ssm_amd_last_error(void) { return ssm::g_last_error; }

extern "C" const char *ssm_amd_status_string(int status) {
  switch (status) {
    case SSM_OK: return "ok";
    case SSM_ERR_NULL_POINTER: return "required pointer is NULL";
    case SSM_ERR_BAD_SHAPE: return "invalid or inconsistent sizes";
    case SSM_ERR_BAD_DTYPE: return "unsupported dtype";
    case SSM_ERR_BAD_KIND: return "unsupported layout / kind / activation";
    case SSM_ERR_ALIGNMENT: return "misaligned pointer";
    case SSM_ERR_TOO_LARGE: return "size exceeds kernel indexing range";
    case SSM_ERR_LAUNCH: return "HIP launch failed";
    case SSM_ERR_WORKSPACE: return "workspace missing or too small";
    default: return "unknown status";
  }
}
