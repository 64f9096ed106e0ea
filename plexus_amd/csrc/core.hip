// Library-wide pieces of libplexus_hip: version, status strings, thread-local error text.
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace {
thread_local char g_last_error[512] = "";
}

namespace plx {
void set_last_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}
}  // namespace plx

extern "C" {

int plx_version(void) { return 100; }

const char *plx_error_string(int status)
{
    switch (status) {
        case PLX_OK: return "ok";
        case PLX_ERR_INVALID: return "invalid argument";
        case PLX_ERR_HIP: return "HIP runtime error";
        case PLX_ERR_WORKSPACE: return "workspace missing or too small";
        case PLX_ERR_UNSUPPORTED: return "unsupported shape";
        case PLX_ERR_NOMEM: return "out of memory";
        default: return "unknown status";
    }
}

const char *plx_last_error(void) { return g_last_error; }

}  // extern "C"
