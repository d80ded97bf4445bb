// Error bookkeeping shared by the entry points of libflashgs_hip.so.
#include "fgs_internal.h"

#include <stdarg.h>
#include <stdio.h>

namespace fgs {
namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t st, const char* what)
{
    if (st == hipSuccess) return FGS_OK;
    (void)hipGetLastError();   // clear the sticky status so that later calls start clean
    return fail(FGS_E_HIP, "%s: %s", what, hipGetErrorString(st));
}

} // namespace fgs

extern "C" const char* fgs_last_error(void) { return fgs::g_last_error; }

extern "C" int fgs_abi_version(void) { return FGS_ABI_VERSION; }
