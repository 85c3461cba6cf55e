// Thread-local error text and library identification.
#include <stdarg.h>

#include "common.h"

namespace ms {
namespace {
thread_local char g_error[512] = "";
}
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
}  // namespace ms

extern "C" const char *ms_last_error(void) { return ms::g_error; }
extern "C" int ms_version(void) { return 100; }
