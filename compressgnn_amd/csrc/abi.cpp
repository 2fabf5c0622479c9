// Error reporting shared by the entry points of the device library.
#include <cstdarg>
#include <cstdio>

#include "compressgnn_abi.h"

namespace cgnn {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

}  // namespace cgnn

extern "C" const char *cgnn_last_error(void) { return cgnn::g_error; }
extern "C" const char *cgnn_version(void) { return "compressgnn-hip 0.1 (gfx950)"; }
