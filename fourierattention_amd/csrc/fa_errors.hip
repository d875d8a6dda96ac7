// Error bookkeeping shared by every entry point of the C ABI.
#include "fa_common.h"

#include <string.h>

namespace {
thread_local char g_last_error[512] = "";
}

void fa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int fa_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fa_set_error("%s: %s", what, hipGetErrorString(e));
    return FA_ERR_LAUNCH;
  }
  return FA_OK;
}

extern "C" const char* fa_last_error_string(void) { return g_last_error; }
extern "C" int fa_abi_version(void) { return 3; }
extern "C" size_t fa_decode_args_size(void) { return sizeof(fa_decode_args); }
