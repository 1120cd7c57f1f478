// Thread-local error text behind mi355_last_error().
#include <cstdarg>
#include <cstdio>

#include "mi355_qlinear.h"

namespace mi355 {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

void clear_error() { g_error[0] = '\0'; }
}  // namespace mi355

extern "C" const char* mi355_last_error(void) { return mi355::g_error; }
extern "C" int mi355_qlinear_abi_version(void) { return MI355_QLINEAR_ABI_VERSION; }
