#include "errors.h"

#include <cstdarg>
#include <cstdio>

#include "../../include/smat.h"

namespace smat {
static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
} // namespace smat

extern "C" const char *smat_last_error(void) { return smat::g_err; }
