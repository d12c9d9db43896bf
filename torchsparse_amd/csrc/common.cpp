#include "common.h"

#include <cstring>

namespace tsmi {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = 0; }

}  // namespace tsmi

extern "C" const char *tsmi_last_error(void) { return tsmi::g_error; }
extern "C" int tsmi_version(void) { return 1; }
