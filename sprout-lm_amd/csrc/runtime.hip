// Error reporting of the C interface.
#include <stdarg.h>
#include <string.h>

#include "common.h"
#include "sprout_hip.h"

namespace sprout {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return 1;
  }
  return 0;
}
}  // namespace sprout

extern "C" const char* sp_last_error() { return sprout::g_error; }
extern "C" int sp_version() { return 1; }
