// Error string plumbing and version of the C ABI.
#include "common.h"

namespace mole {
static thread_local char g_err[512] = "";
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
}  // namespace mole

extern "C" int mole_version(void) { return 100; }
extern "C" const char *mole_last_error_string(void) { return mole::g_err; }
