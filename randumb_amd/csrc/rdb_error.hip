// Error bookkeeping and library identification for librandumb_hip.
#include <stdarg.h>
#include <stdio.h>
#include <unistd.h>

#include <atomic>
#include <random>

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

// ----------------------------------------------------------------------------------------------- waits that gave up
// Counter of blocks that gave up waiting for blocks of their own launch (rdb_common.hpp: await_tags); every device that runs
// the library holds its own copy, zero when the library is loaded there.  In host code the name is only a handle: the
// address is asked for once per device, with that device current, and kept.
static __device__ unsigned int rdb_sync_giveup_count;

int sync_giveups_ptr(unsigned int **out)
{
    static unsigned int *ptrs[64] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error((int)e, "give-up counter: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return set_error(RDB_E_UNSUPPORTED, "give-up counter: device index %d outside 0..63", dev);
    unsigned int *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        void *v = nullptr;
        e = hipGetSymbolAddress(&v, HIP_SYMBOL(rdb_sync_giveup_count));
        if (e != hipSuccess || !v) return set_error(e != hipSuccess ? (int)e : RDB_E_UNSUPPORTED, "give-up counter: hipGetSymbolAddress: %s", hipGetErrorString(e));
        p = static_cast<unsigned int *>(v);
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);   // every thread that gets here asks for the same address
    }
    *out = p;
    return RDB_OK;
}

// A tag no other launch of any process is likely ever to have written where a launch's slots lie: a counter that starts at a
// random 64-bit value.
unsigned long long next_sync_tag()
{
    static std::atomic<unsigned long long> counter{[] {
        std::random_device rd;
        return ((unsigned long long)rd() << 32) ^ (unsigned long long)rd() ^ ((unsigned long long)getpid() << 17);
    }()};
    unsigned long long v = counter.fetch_add(1) + 1;
    return v ? v : counter.fetch_add(1) + 1;
}

static int g_one_launch = 1;
int one_launch_mode() { return __atomic_load_n(&g_one_launch, __ATOMIC_RELAXED); }

}  // namespace rdb

extern "C" int rdb_abi_version(void) { return 8; }

extern "C" int rdb_set_one_launch(int mode)
{
    return __atomic_exchange_n(&rdb::g_one_launch, mode ? 1 : 0, __ATOMIC_RELAXED);
}

extern "C" int rdb_sync_giveups_async(uint32_t *host_count, void *stream)
{
    if (!host_count) return rdb::set_error(RDB_E_NULL, "rdb_sync_giveups_async: host_count is NULL");
    unsigned int *p = nullptr;
    if (int rc = rdb::sync_giveups_ptr(&p)) return rc;
    hipError_t e = hipMemcpyAsync(host_count, p, sizeof(uint32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e != hipSuccess) return rdb::set_error((int)e, "rdb_sync_giveups_async: hipMemcpyAsync: %s", hipGetErrorString(e));
    return RDB_OK;
}

extern "C" int rdb_sync_giveups(uint32_t *count, void *stream)
{
    if (!count) return rdb::set_error(RDB_E_NULL, "rdb_sync_giveups: count is NULL");
    unsigned int *p = nullptr;
    if (int rc = rdb::sync_giveups_ptr(&p)) return rc;
    hipError_t e = hipMemcpyAsync(count, p, sizeof(uint32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return rdb::set_error((int)e, "rdb_sync_giveups: %s", hipGetErrorString(e));
    return RDB_OK;
}
extern "C" const char *rdb_last_error_string(void) { return rdb::g_err; }
