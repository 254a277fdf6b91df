// Error reporting shared by every entry point.  An entry point returns 0 on
// success; otherwise `ix_last_error()` holds the reason for the calling thread.
#include "common.h"

static thread_local std::string g_error;

void ix_set_error(const std::string& msg) { g_error = msg; }

int ix_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_error = std::string(what) + ": " + hipGetErrorString(e);
    return 1;
  }
  return 0;
}

extern "C" const char* ix_last_error() { return g_error.c_str(); }

extern "C" int ix_abi_version() { return 1; }
