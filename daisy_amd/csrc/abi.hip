// Error state and version of the C ABI.
#include "common.h"

namespace daisy {

static thread_local char g_err[512] = {0};

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

}  // namespace daisy

extern "C" const char* daisy_last_error(void) { return daisy::g_err; }

extern "C" int daisy_abi_version(void) { return 5; }
