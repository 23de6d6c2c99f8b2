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

// Raises a kernel's dynamic-LDS limit to `smem` bytes on the current device, once: the driver call is only made when this
// (kernel, device) pair has not been given at least that much before.  A small lock-free table; a pair that finds it full
// simply makes the driver call every time.
int reserve_lds(const void *kernel, size_t smem, const char *name)
{
    struct Slot {
        const void *fn;
        int dev;
        size_t smem;
    };
    static Slot table[256];
    static int used = 0;   // slots [0, used) are complete; entries are only ever appended or grown
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = -1;
    const int n = __atomic_load_n(&used, __ATOMIC_ACQUIRE);
    for (int i = 0; i < n; ++i)
        if (table[i].fn == kernel && table[i].dev == dev) {
            if (__atomic_load_n(&table[i].smem, __ATOMIC_RELAXED) >= smem) return RDB_OK;
            hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return set_error((int)e, "%s: cannot reserve %zu bytes of LDS: %s", name, smem, hipGetErrorString(e));
            __atomic_store_n(&table[i].smem, smem, __ATOMIC_RELAXED);
            return RDB_OK;
        }
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return set_error((int)e, "%s: cannot reserve %zu bytes of LDS: %s", name, smem, hipGetErrorString(e));
    static int lock = 0;   // appends are rare (once per kernel and device): a spin lock keeps them apart
    while (__atomic_exchange_n(&lock, 1, __ATOMIC_ACQUIRE)) {
    }
    const int m = __atomic_load_n(&used, __ATOMIC_RELAXED);
    if (m < 256 && dev >= 0) {
        table[m].fn = kernel;
        table[m].dev = dev;
        table[m].smem = smem;
        __atomic_store_n(&used, m + 1, __ATOMIC_RELEASE);
    }
    __atomic_store_n(&lock, 0, __ATOMIC_RELEASE);
    return RDB_OK;
}

int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return RDB_OK;
    return set_error((int)e, "%s: %s", what, hipGetErrorString(e));
}

// Compute units of the current device; 256 when there is none (size queries without a GPU).
int num_compute_units()
{
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace rdb

extern "C" int rdb_abi_version(void) { return 6; }
extern "C" const char *rdb_last_error_string(void) { return rdb::g_err; }
