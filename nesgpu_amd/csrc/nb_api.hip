// Error reporting and version of libnesbin.so.
#include <cstdarg>
#include <cstdio>

#include "nb_common.hpp"

namespace nb {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return NB_OK;
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return NB_ERR_HIP_BASE + (int)e;
}

}  // namespace nb

extern "C" int nb_version(void) { return 100; }
extern "C" const char *nb_last_error_string(void) { return nb::g_err; }
