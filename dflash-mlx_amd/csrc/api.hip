// ABI bookkeeping of libdflash_mi355.so: version and per-thread error text.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "dflash_common.h"

namespace dflash {
namespace {
thread_local char g_error[512] = "";
std::atomic<int> g_options[DFLASH_OPT_COUNT];
}

int option(int which) { return g_options[which].load(std::memory_order_relaxed); }

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace dflash

extern "C" int dflash_abi_version(void) { return DFLASH_ABI_VERSION; }

extern "C" const char* dflash_last_error(void) { return dflash::g_error; }

extern "C" int dflash_set_option(int option, int value) {
  DFLASH_REQUIRE(option >= 0 && option < DFLASH_OPT_COUNT && value >= 0, DFLASH_ERR_ARG,
                 "dflash_set_option: option %d, value %d", option, value);
  dflash::g_options[option].store(value, std::memory_order_relaxed);
  return DFLASH_OK;
}

extern "C" int dflash_get_option(int option) {
  DFLASH_REQUIRE(option >= 0 && option < DFLASH_OPT_COUNT, DFLASH_ERR_ARG, "dflash_get_option: option %d", option);
  return dflash::option(option);
}

extern "C" int dflash_qmm_error(const void* workspace, uint32_t* word_host, void* stream) {
  DFLASH_REQUIRE(workspace && word_host, DFLASH_ERR_ARG, "dflash_qmm_error: null argument");
  DFLASH_HIP_OK(hipStreamSynchronize((hipStream_t)stream));
  DFLASH_HIP_OK(hipMemcpy(word_host, (const char*)workspace + DFLASH_QMM_ERROR_OFFSET, sizeof(uint32_t),
                          hipMemcpyDeviceToHost));
  return DFLASH_OK;
}
