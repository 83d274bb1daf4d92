// ABI bookkeeping of libdflash_mi355.so: version and per-thread error text.
#include <stdarg.h>
#include <stdio.h>

#include "dflash_common.h"

namespace dflash {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace dflash

extern "C" int dflash_abi_version(void) { return DFLASH_ABI_VERSION; }

extern "C" const char* dflash_last_error(void) { return dflash::g_error; }
