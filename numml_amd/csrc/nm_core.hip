// Error reporting and version of libnumml_hip.so.
#include "nm_common.hpp"

#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_last_error[512] = "";
}

namespace nm {
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}
}  // namespace nm

extern "C" int nm_version(void) { return 1000; }

extern "C" const char *nm_last_error(void) { return g_last_error; }
