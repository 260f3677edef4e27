// Error state and ABI version of liblbi_hip.so.
#include "lbi_common.h"

#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_error[512] = "";
}

namespace lbi {

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}

void clear_error() { g_error[0] = '\0'; }

}  // namespace lbi

extern "C" int lbi_abi_version(void) { return 9; }

extern "C" const char* lbi_last_error(void) { return g_error; }
