// Thread-local error reporting for the C ABI.
#include "stmoe_common.h"

namespace stmoe {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(STMOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return STMOE_OK;
}

}  // namespace stmoe

extern "C" const char* stmoe_last_error(void) { return stmoe::g_last_error; }
extern "C" int stmoe_abi_version(void) { return 1; }
