// Shared device helpers for librandumb_hip: Squirrel5 noise, bf16 conversion, MFMA fragments, errors.
// gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/randumb_hip.h"

namespace rdb {

// ----------------------------------------------------------------------------------------------- errors
int set_error(int code, const char *fmt, ...);  // records the message for rdb_last_error_string, returns code
int check_launch(const char *what);             // hipGetLastError -> positive code + message
int reserve_lds(const void *kernel, size_t smem, const char *name);  // dynamic-LDS limit of a kernel, set once per device

// ----------------------------------------------------------------------------------------------- noise
// Squirrel5 constants and the row/column mixing prime (reference: src/rten_cpp/RandumbTensor.py:140-145,
// src/rten_cpp/csrc/cuda/rten.cu:13-18).
constexpr uint32_t SQ5_N1 = 0xd2a80a3fu;
constexpr uint32_t SQ5_N2 = 0xa884f197u;
constexpr uint32_t SQ5_N3 = 0x6C736F4Bu;
constexpr uint32_t SQ5_N4 = 0xB79F3ABBu;
constexpr uint32_t SQ5_N5 = 0x1b56c4f5u;
constexpr uint32_t PRIME = 198491317u;
// (PRIME*n + m)*N1 + seed == n*PN1 + m*N1 + seed (mod 2^32): lets a loop over n or m advance the first
// round with one add instead of a multiply.
constexpr uint32_t PN1 = (uint32_t)((uint64_t)PRIME * (uint64_t)SQ5_N1);

// Rounds after "b = idx*N1 + seed" (reference: RandumbTensor.py:151-159).
__device__ __forceinline__ uint32_t sq5_tail(uint32_t b)
{
    b ^= (b >> 9);
    b += SQ5_N2;
    b ^= (b >> 11);
    b *= SQ5_N3;
    b ^= (b >> 13);
    b += SQ5_N4;
    b ^= (b >> 15);
    b *= SQ5_N5;
    b ^= (b >> 17);
    return b;
}

__device__ __forceinline__ uint32_t sq5_bits(uint32_t idx, uint32_t seed) { return sq5_tail(idx * SQ5_N1 + seed); }

// int32 reinterpretation -> fp32 (round to nearest even) -> exact scale by 2^-31
// (reference: RandumbTensor.py:162-163; fp32(1/0x7FFFFFFF) == 2^-31).
__device__ __forceinline__ float sq5_unit(uint32_t bits) { return (float)(int32_t)bits * 4.656612873077392578125e-10f; }

__device__ __forceinline__ float noise1d(uint32_t idx, uint32_t seed) { return sq5_unit(sq5_bits(idx, seed)); }
__device__ __forceinline__ float noise2d(uint32_t n, uint32_t m, uint32_t seed)
{
    return sq5_unit(sq5_bits(PRIME * n + m, seed));
}
// First-round value for (n, m): pass to sq5_tail.  first(n, m+1) = first(n, m) + N1; first(n+1, m) = first(n, m) + PN1.
__device__ __forceinline__ uint32_t sq5_first(uint32_t n, uint32_t m, uint32_t seed) { return n * PN1 + m * SQ5_N1 + seed; }

// ----------------------------------------------------------------------------------------------- bf16
typedef uint16_t bf16_t;  // storage type
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi)
{
    f32x2 v = {lo, hi};
    bf16x2 r = __builtin_convertvector(v, bf16x2);  // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return (bf16_t)(f32x2_to_bf16x2(f, 0.0f) & 0xffffu); }

template <typename T> struct elem;
template <> struct elem<float> {
    static constexpr int dtype = RDB_F32;
    __device__ static __forceinline__ float load(const float *p) { return *p; }
    __device__ static __forceinline__ void store(float *p, float v) { *p = v; }
    __device__ static __forceinline__ float round(float v) { return v; }
};
template <> struct elem<bf16_t> {
    static constexpr int dtype = RDB_BF16;
    __device__ static __forceinline__ float load(const bf16_t *p) { return bf16_to_f32(*p); }
    __device__ static __forceinline__ void store(bf16_t *p, float v) { *p = f32_to_bf16(v); }
    __device__ static __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

// Reads element i of a buffer whose dtype is only known at run time.
__device__ __forceinline__ float load_as_f32(const void *p, int dtype, int64_t i)
{
    return dtype == RDB_BF16 ? bf16_to_f32(((const bf16_t *)p)[i]) : ((const float *)p)[i];
}

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ----------------------------------------------------------------------------------------------- timeline stamps
// RDB_STAMP(slot), slot 0..3, records when thread 0 of a block passes a point of a kernel.  Compiled out of the library.  A
// timing harness defines RDB_STAMPS and a __device__ pointer rdb_stamp_buf before including the kernel sources and then
// finds, per block, 4 kernels x 4 slots of two counters: the constant-rate wall clock (comparable across compute units) and
// the shader clock.  Which of the 4 kernels a launch is, the harness says with an expression RDB_STAMP_KERNEL_ID over the
// launch geometry (no extra registers or LDS in the kernels, so their occupancy is that of the library's build).
// 16-byte store of data that the kernel which writes it does not read again (it is for the next launch, on other dies):
// non-temporal, so the line does not wait dirty in this die's L2 for the write-back at the end of the kernel.
template <class V> __device__ __forceinline__ void store_stream(V *dst, const V &v)
{
#ifdef RDB_NO_STREAM_STORES
    *dst = v;
#else
    __builtin_nontemporal_store(v, dst);
#endif
}

// ----------------------------------------------------------------------------------------------- producer -> consumer blocks of one launch
// Blocks of one launch that consume what earlier blocks of the same launch produce: a producer publishes a 64-bit tag, unique
// to the launch, in a slot of its own when its output is in memory; a consumer polls the slots it depends on.  Hardware
// queues hand out the blocks of a launch in index order (per die), so a consumer that only waits for blocks with lower
// indices cannot starve them.  That order is what the hardware is seen to do, not something its documentation promises, so
// the wait is bounded: after `polls` polls (SYNC_SPIN_LIMIT: a fraction of a second) the consumer gives up.  A block that
// gives up never computes on what happens to be in memory: it counts itself in the library's per-device give-up counter
// (which the host reads: rdb_sync_giveups), sets bit 1 of *err when the caller has such a word, and its caller fills the
// block's share of the output with NaN and leaves.
//
// The dies' L2 caches are not coherent with each other, and the fences that make them so (write back / invalidate a whole
// L2) cost microseconds per block.  So the data that passes from producer to consumer goes around them instead: stored and
// loaded with device scope (SCOPE_DEVICE below: write-through, and read from memory), as the tags are.
constexpr int SYNC_SPIN_LIMIT = 1 << 17;
constexpr int SCOPE_DEVICE = 16;   // cache-policy argument of the raw buffer loads and stores: sc1

// What a waiting block needs besides its slots: how long to wait and where to report that it gave up.
struct SyncWait {
    unsigned int *err;       // NULL, or a word of the caller's state: bit 1 is set by a block that gave up
    unsigned int *giveups;   // the library's counter of such blocks on this device
    int polls;               // bound of the wait
};

// Device address of the give-up counter of the current device (rdb_error.hip); one per device, zero when the library loads.
int sync_giveups_ptr(unsigned int **out);
// The tag of a launch (never 0).
unsigned long long next_sync_tag();
// 1: the one-launch forms run where they apply; 0: producers and consumers always as separate launches (rdb_set_one_launch).
int one_launch_mode();

// All threads of the block call this after their last store (with SCOPE_DEVICE) of the block's output.
__device__ __forceinline__ void publish_tag(unsigned long long *slot, unsigned long long tag)
{
    __builtin_amdgcn_s_waitcnt(0);   // this wave's stores have been acknowledged at their scope
    __syncthreads();                 // ... and every other wave's
    if (threadIdx.x == 0) __hip_atomic_store(slot, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One wave calls this: lanes 0 .. n - 1 (n <= 64) poll slots[0 .. n - 1].  Returns false after the poll limit: the caller must
// then poison its output instead of computing it.  Loads of the producers' data that follow must use SCOPE_DEVICE.
__device__ __forceinline__ bool await_tags(const unsigned long long *slots, int n, unsigned long long tag, const SyncWait &w)
{
    const int lane = threadIdx.x & 63;
    const unsigned long long *mine = slots + (lane < n ? lane : 0);
    for (int it = 0; it < w.polls; ++it) {
        const unsigned long long v = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__all(v == tag)) return true;
        __builtin_amdgcn_s_sleep(20);
    }
    if (lane == 0) {
        if (w.err) atomicOr(w.err, 2u);
        atomicAdd(w.giveups, 1u);
    }
    return false;
}

// The same wave calls this once its wait has succeeded.  A launch recorded in a graph runs again with the tag it was recorded
// with, so the slots must not still hold it then: every consumer of the n slots counts itself in `counter`, and the last of
// the `consumers` (all of them are past their wait by then) clears the slots.  The counter is set to zero by one of the
// producers of these slots before it publishes its tag (store it before the call of publish_tag).
__device__ __forceinline__ void release_tags(unsigned long long *slots, int n, unsigned int *counter, int consumers)
{
    const int lane = threadIdx.x & 63;
    unsigned int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = (unsigned int)__builtin_amdgcn_readfirstlane((int)old);
    if (old == (unsigned int)(consumers - 1) && lane < n) __hip_atomic_store(slots + lane, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

#ifdef RDB_STAMPS
#ifndef RDB_STAMP_KERNEL_ID
#define RDB_STAMP_KERNEL_ID 0
#endif
#define RDB_STAMP(slot)                                                                                                  \
    do {                                                                                                                 \
        if (threadIdx.x == 0 && rdb_stamp_buf) {                                                                         \
            const size_t at_ = ((size_t)blockIdx.x * 16 + (RDB_STAMP_KERNEL_ID) * 4 + (slot)) * 2;                       \
            rdb_stamp_buf[at_] = wall_clock64();                                                                         \
            rdb_stamp_buf[at_ + 1] = clock64();                                                                          \
        }                                                                                                                \
    } while (0)
#else
#define RDB_STAMP(slot) ((void)0)
#endif

}  // namespace rdb
