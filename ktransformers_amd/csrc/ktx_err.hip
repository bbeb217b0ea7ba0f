// ktx_err.hip — the per-thread error slot behind ktx_last_error(): every entry point of the C ABI returns 0 or stores a message
// here and returns -1 (KTX_REQUIRE / KTX_HIP in ktx_common.h).  A source of its own so that a library built from a subset of the
// kernel files (libktx_seq.so) carries it too.
#include "ktx_common.h"

std::string& ktx_err_slot() {
  static thread_local std::string s;
  return s;
}
int ktx_fail(const std::string& msg) {
  ktx_err_slot() = msg;
  return -1;
}
extern "C" const char* ktx_last_error(void) { return ktx_err_slot().c_str(); }
