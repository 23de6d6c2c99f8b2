// Error bookkeeping and library identification for librandumb_hip.
#include <stdarg.h>
#include <stdio.h>

#include "rdb_common.hpp"

namespace rdb {

static thread_local char g_err[512] = "no error";

int set_error(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return RDB_OK;
    return set_error((int)e, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace rdb

extern "C" int rdb_abi_version(void) { return 4; }
extern "C" const char *rdb_last_error_string(void) { return rdb::g_err; }
