// Thread-local error text, library identification, per-device kernel attribute cache.
#include <stdarg.h>

#include <map>
#include <mutex>
#include <utility>

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

hipError_t set_max_dynamic_lds(const void *fn, int bytes) {
    static std::mutex mu;
    static std::map<std::pair<const void *, int>, int> done;   // (kernel, device) -> size already set
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mu);
    int &have = done[std::make_pair(fn, dev)];
    if (have >= bytes) return hipSuccess;
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) have = bytes;
    return e;
}
}  // namespace ms

extern "C" const char *ms_last_error(void) { return ms::g_error; }
extern "C" int ms_version(void) { return 103; }
