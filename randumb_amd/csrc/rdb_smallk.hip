// Fused linear layer, matrix-coef + fp32, small coefficient dimension and few tokens (the GEMV-like regime): factored
// algorithm on the vector ALU.
//
// With k <= 64 and a handful of tokens the layer moves almost no data (x, C, y) and does almost no arithmetic once W = C . N
// is used associatively; what remains is the hash of N, in_f * k values per token tile:
//   forward  z = x . N^T [T x k],  y = z . C^T (+ bias)
//   dx       t = dy . C  [T x k],  dx = t . N
//   dcoef    z as above,           dC = dy^T . z
// Everything is fp32 FMA with partial sums combined in a fixed order (no atomics): results are bit-reproducible.
// Replaces materialize() + dense product (src/rten_cpp/RandumbTensor.py:942-946) and MmBackward's dW followed by
// materialize_bwd (RandumbTensor.py:979-990, 304-359) in the regime where a stored-W product would be bound by reading W.
#include "rdb_common.hpp"

namespace rdb {

constexpr int SK_TT = 8;    // tokens per block of the contracting kernel
constexpr int SK_ET = 16;   // tokens per block of the expanding kernel
constexpr int SK_MAX_K = 64;

// sum over the partial matrices p[ch][idx], ch = 0 .. nchunk-1, in chunk order; loads issued eight at a time
__device__ __forceinline__ float sum_partials(const float *__restrict__ p, int64_t stride, int nchunk)
{
    float v = 0.0f;
    for (int c0 = 0; c0 < nchunk; c0 += 8) {
        float l[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) l[u] = p[(int64_t)((c0 + u < nchunk) ? c0 + u : nchunk - 1) * stride];  // always a valid address
#pragma unroll
        for (int u = 0; u < 8; ++u) v += (c0 + u < nchunk) ? l[u] : 0.0f;
    }
    return v;
}

// out[t, m] = sum_j src[t, j] * B(j, m),  B(j, m) = noise(PRIME*j + m) (HASH) or coef[j, m]; j runs over J = in_f or out_f.
// Block = 8 tokens x one chunk of 256 values of j (blockIdx.y), so that even a single token spreads the hash over many
// compute units; thread = (m % 16, one of 16 interleaved slices of the chunk); the source rows go through LDS (coalesced
// loads, broadcast reads); slices meet in LDS in slice order.  The block writes a partial result, out[chunk][t][m]; the
// expanding kernel adds the chunks up in chunk order while it loads them.
struct SkContract {
    float *out;          // [chunks][T][k] partial sums
    const float *src;    // [T x J], leading dimension ld_src
    int64_t ld_src;
    const float *coef;   // [J x k] (not HASH)
    int T, J, k;
    uint32_t seed;
};

// bx: token tile, by: chunk of 256 values of j.  The partial sums are stored at device scope: blocks of the same launch on
// another die may be the ones that read them (smallk_fused_kernel).
template <bool HASH> __device__ __forceinline__ void smallk_contract_block(const SkContract &p, int bx, int by)
{
    constexpr int JC = 256, MC = SK_MAX_K / 16;
    __shared__ float xs[SK_TT][JC];
    __shared__ float red[16][SK_TT][16];
    float *__restrict__ out = p.out;
    const float *__restrict__ src = p.src;
    const float *__restrict__ coef = p.coef;
    const int64_t lds_src = p.ld_src;
    const int T = p.T, J = p.J, k = p.k;
    const uint32_t seed = p.seed;
    const int tid = threadIdx.x, m16 = tid & 15, slice = tid >> 4;
    const int t0 = bx * SK_TT;
    float acc[MC][SK_TT];
#pragma unroll
    for (int c = 0; c < MC; ++c)
#pragma unroll
        for (int tt = 0; tt < SK_TT; ++tt) acc[c][tt] = 0.0f;
    {
        const int jc = by * JC;
#pragma unroll
        for (int tt = 0; tt < SK_TT; ++tt) xs[tt][tid] = (t0 + tt < T && jc + tid < J) ? src[(int64_t)(t0 + tt) * lds_src + jc + tid] : 0.0f;
        __syncthreads();
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            const int m = c * 16 + m16;
            if (c * 16 < k) {  // uniform
                uint32_t first = sq5_first((uint32_t)(jc + slice), (uint32_t)m, seed);
                for (int jj = 0; jj < JC / 16; ++jj, first += 16u * PN1) {
                    const int j = jc + slice + 16 * jj;
                    // no branches in here: out-of-range (j, m) read a valid address and are zeroed by a select
                    float b = HASH ? sq5_unit(sq5_tail(first)) : coef[(int64_t)(j < J ? j : J - 1) * k + (m < k ? m : k - 1)];
                    b = (m < k && j < J) ? b : 0.0f;
#pragma unroll
                    for (int tt = 0; tt < SK_TT; ++tt) acc[c][tt] = fmaf(xs[tt][slice + 16 * jj], b, acc[c][tt]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < MC; ++c) {
        if (c * 16 >= k) break;
#pragma unroll
        for (int tt = 0; tt < SK_TT; ++tt) red[slice][tt][m16] = acc[c][tt];
        __syncthreads();
        if (tid < SK_TT * 16) {
            const int tt = tid >> 4, m = c * 16 + m16;
            float s = 0.0f;
#pragma unroll
            for (int sl = 0; sl < 16; ++sl) s += red[sl][tt][m16];
            if (t0 + tt < T && m < k) __hip_atomic_store(out + ((int64_t)by * T + t0 + tt) * k + m, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    }
}

template <bool HASH> __global__ __launch_bounds__(256) void smallk_contract_kernel(SkContract p) { smallk_contract_block<HASH>(p, blockIdx.x, blockIdx.y); }

// out[t, c] = sum_m src[t, m] * B(c, m) (+ bias[c]),  B(c, m) = noise(PRIME*c + m) (HASH) or coef[c, m]; c runs over the
// cols = in_f or out_f.  Block = 256 columns x 16 tokens; a thread owns one column and keeps its 16 B values in registers.
// src holds `nchunk` partial matrices [T x k] (from the contracting kernel), added up here in chunk order.
struct SkExpand {
    float *out;          // [T x cols], leading dimension ld_out
    int64_t ld_out;
    const float *src;    // [nchunk][T][k] partial sums
    int nchunk;
    const float *coef;   // [cols x k] (not HASH)
    const float *bias;   // [cols] or NULL
    int T, cols, k;
    uint32_t seed;
    // NULL, or slots [token tiles of SK_TT][nchunk] that contracting blocks of the same launch set to sync_tag; sync_count: one
    // counter per SK_ET tokens of the expanding blocks that have seen them (sync_consumers of them: the last clears the slots)
    unsigned long long *sync;
    unsigned long long sync_tag;
    SyncWait sync_wait;
    unsigned int *sync_count;
    int sync_consumers;
};

// bx: block of 256 columns, by: block of SK_ET tokens.
template <bool HASH> __device__ __forceinline__ void smallk_expand_block(const SkExpand &p, int bx, int by)
{
    __shared__ __align__(16) float s[SK_ET][SK_MAX_K];
    float *__restrict__ out = p.out;
    const float *__restrict__ src = p.src;
    const float *__restrict__ coef = p.coef;
    const float *__restrict__ bias = p.bias;
    const int64_t ld_out = p.ld_out;
    const int nchunk = p.nchunk, T = p.T, cols = p.cols, k = p.k;
    const uint32_t seed = p.seed;
    const int tid = threadIdx.x;
    const int c = bx * 256 + tid, t0 = by * SK_ET;
    // this thread's first 16 values of B: fetched (or hashed) before anything is waited for
    float b0[16];
    {
        const int cc = c < cols ? c : cols - 1;
#pragma unroll
        for (int m = 0; m < 16; ++m) {  // branch-free: a column from k on reads a valid address and becomes 0
            const float v = HASH ? sq5_unit(sq5_tail(sq5_first((uint32_t)cc, (uint32_t)m, seed))) : coef[(int64_t)cc * k + ((m < k) ? m : k - 1)];
            b0[m] = (m < k) ? v : 0.0f;
        }
    }
    if (p.sync) {   // the partial sums of these tokens come from earlier blocks of this launch
        __shared__ int verdict;
        if (tid < 64) {
            const int tile0 = t0 / SK_TT, tiles = (T + SK_TT - 1) / SK_TT;
            const int ntile = (tile0 + SK_ET / SK_TT <= tiles) ? SK_ET / SK_TT : tiles - tile0;
            unsigned long long *slots = p.sync + (int64_t)tile0 * nchunk;
            const bool there = await_tags(slots, ntile * nchunk, p.sync_tag, p.sync_wait);
            if (there) release_tags(slots, ntile * nchunk, p.sync_count + by, p.sync_consumers);
            if (tid == 0) verdict = there ? 1 : 0;
        }
        __syncthreads();
        if (verdict == 0) {   // gave up: the block's share of the output becomes NaN, never a sum of whatever is in memory
            if (c < cols)
                for (int tt = 0; tt < SK_ET; ++tt)
                    if (t0 + tt < T) out[(int64_t)(t0 + tt) * ld_out + c] = __uint_as_float(0x7fc00000u);
            return;
        }
    }
    // s = sum of the partial matrices in chunk order; columns from k on take part as zeros.  A thread owns up to 4 entries
    // and keeps the loads of 8 chunks of all of them in flight at once: the kernel is a chain of memory latencies otherwise.
    {
        constexpr int PER = SK_ET * SK_MAX_K / 256;
        float v[PER];
        const float *ptr[PER];
        bool ok[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + 256 * i, tt = e / k, m = e % k;   // entries e < SK_ET * k, row-major over (tt, m < k)
            v[i] = 0.0f;
            ok[i] = e < SK_ET * k && t0 + tt < T;
            ptr[i] = ok[i] ? src + (int64_t)(t0 + tt) * k + m : src;   // always a valid address
        }
        const int64_t stride = (int64_t)T * k;
        for (int c0 = 0; c0 < nchunk; c0 += 8) {
            float l[PER][8];
#pragma unroll
            for (int i = 0; i < PER; ++i)
#pragma unroll
                for (int u = 0; u < 8; ++u)   // device scope: possibly written by another die during this launch
                    l[i][u] = __hip_atomic_load(ptr[i] + (int64_t)((c0 + u < nchunk) ? c0 + u : nchunk - 1) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int i = 0; i < PER; ++i)
#pragma unroll
                for (int u = 0; u < 8; ++u) v[i] += (ok[i] && c0 + u < nchunk) ? l[i][u] : 0.0f;
        }
        for (int e = tid; e < SK_ET * SK_MAX_K; e += 256) s[e / SK_MAX_K][e % SK_MAX_K] = 0.0f;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = tid + 256 * i;
            if (e < SK_ET * k) s[e / k][e % k] = v[i];
        }
    }
    __syncthreads();
    if (c >= cols) return;
    float acc[SK_ET];
#pragma unroll
    for (int tt = 0; tt < SK_ET; ++tt) acc[tt] = 0.0f;
    for (int mc = 0; mc < k; mc += 16) {
        float b[16];
        if (mc == 0) {
#pragma unroll
            for (int m = 0; m < 16; ++m) b[m] = b0[m];
        } else {
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                const float v = HASH ? sq5_unit(sq5_tail(sq5_first((uint32_t)c, (uint32_t)(mc + m), seed)))
                                     : coef[(int64_t)c * k + ((mc + m < k) ? mc + m : k - 1)];
                b[m] = (mc + m < k) ? v : 0.0f;
            }
        }
        // mc <= 48 and m <= 15: always inside the 64 columns of s
#pragma unroll
        for (int tt = 0; tt < SK_ET; ++tt) {
            const f32x4 *row = reinterpret_cast<const f32x4 *>(&s[tt][mc]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 sv = row[q];
                acc[tt] = fmaf(sv[0], b[4 * q], acc[tt]);
                acc[tt] = fmaf(sv[1], b[4 * q + 1], acc[tt]);
                acc[tt] = fmaf(sv[2], b[4 * q + 2], acc[tt]);
                acc[tt] = fmaf(sv[3], b[4 * q + 3], acc[tt]);
            }
        }
    }
    const float bv = bias ? bias[c] : 0.0f;
#pragma unroll
    for (int tt = 0; tt < SK_ET; ++tt)
        if (t0 + tt < T) out[(int64_t)(t0 + tt) * ld_out + c] = acc[tt] + bv;
}

template <bool HASH> __global__ __launch_bounds__(256) void smallk_expand_kernel(SkExpand p) { smallk_expand_block<HASH>(p, blockIdx.x, blockIdx.y); }

// Both in one launch: the contracting blocks first, each publishing a tag when its partial sums are in memory, then the
// expanding blocks, each waiting for the tags of its 16 tokens' tiles.  At a few tokens the two launches are most of the
// time of the call.
struct SkFused {
    SkContract c;
    SkExpand e;
    unsigned long long *slots;
    unsigned int *counters;   // one per SK_ET tokens, cleared by the contracting block of the group's first tile and chunk 0
    int c_tiles, c_blocks, e_colblocks;
};

template <bool CHASH> __global__ __launch_bounds__(256) void smallk_fused_kernel(SkFused p)
{
    const int b = blockIdx.x;
    if (b < p.c_blocks) {
        const int bx = b % p.c_tiles, by = b / p.c_tiles;
        // a replayed launch carries the tag it was recorded with: should a consumer of an earlier replay have given up, the slot
        // may still hold it (the consumers clear the slots only when all of them got past their wait)
        if (threadIdx.x == 0) __hip_atomic_store(p.slots + (int64_t)bx * p.e.nchunk + by, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        smallk_contract_block<CHASH>(p.c, bx, by);
        if (by == 0 && bx % (SK_ET / SK_TT) == 0 && threadIdx.x == 0)
            __hip_atomic_store(p.counters + bx / (SK_ET / SK_TT), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        publish_tag(p.slots + (int64_t)bx * p.e.nchunk + by, p.e.sync_tag);
    } else {
        const int e = b - p.c_blocks;
        smallk_expand_block<!CHASH>(p.e, e % p.e_colblocks, e / p.e_colblocks);
    }
}

// dC[o, m] = sum_t dy[t, o] * z[t, m].  Block = 256 output rows x one chunk of 16 coefficients; z goes through LDS in tiles
// of 64 tokens; a thread owns one output row and walks the tokens in order.
__global__ __launch_bounds__(256) void smallk_dcoef_kernel(float *__restrict__ dcoef, const float *__restrict__ dy, int64_t lddy,
                                                           const float *__restrict__ z, int nchunk, int T, int out_f, int k)
{
    __shared__ __align__(16) float zs[64][16];
    const int tid = threadIdx.x;
    const int o = blockIdx.x * 256 + tid, mc = blockIdx.y * 16;
    float acc[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] = 0.0f;
    for (int t0 = 0; t0 < T; t0 += 64) {
        for (int e = tid; e < 64 * 16; e += 256) {
            const int tt = e >> 4, m = e & 15;
            zs[tt][m] = (t0 + tt < T && mc + m < k) ? sum_partials(z + (int64_t)(t0 + tt) * k + mc + m, (int64_t)T * k, nchunk) : 0.0f;
        }
        __syncthreads();
        if (o < out_f) {
            const int n = (T - t0 < 64) ? T - t0 : 64;
            for (int tt = 0; tt < n; ++tt) {
                const float g = dy[(int64_t)(t0 + tt) * lddy + o];
#pragma unroll
                for (int m = 0; m < 16; ++m) acc[m] = fmaf(g, zs[tt][m], acc[m]);
            }
        }
        __syncthreads();
    }
    if (o < out_f) {
#pragma unroll
        for (int m = 0; m < 16; ++m)
            if (mc + m < k) dcoef[(int64_t)o * k + mc + m] = acc[m];
    }
}

// ----------------------------------------------------------------------------------------------- host side
// The regime this file is for; AUTO additionally wants it to be the cheaper way.
static bool smallk_ok(const rdb_linear_desc *d)
{
    return d->act_dtype == RDB_F32 && d->coef_dtype == RDB_F32 && d->coef_rows != 0 && d->k > 0 && d->k <= SK_MAX_K && d->tokens > 0 &&
           d->tokens <= 4096 && d->in_f > 0 && d->out_f > 0 && d->in_f < (1 << 30) && d->out_f < (1 << 30);
}
static bool smallk_wanted(const rdb_linear_desc *d)
{
    return d->algo == RDB_ALGO_FACTORED || (d->tokens <= 1024 && d->k * (d->in_f + d->out_f) < d->in_f * d->out_f);
}

// scratch: one partial [tokens x k] fp32 matrix per 256-chunk of the longer of in_f and out_f, then the tag slots of the
// one-launch form (one per token tile and chunk), 8 bytes not in use and a counter per 16 tokens (a waiting block that gives
// up reports to the library's per-device counter: the scratch may be the caller's and gone by the time anybody looks)
static int64_t partial_bytes(const rdb_linear_desc *d)
{
    const int64_t longer = d->in_f > d->out_f ? d->in_f : d->out_f;
    return (cdiv(longer, 256) * d->tokens * d->k * (int64_t)sizeof(float) + 7) / 8 * 8;
}
int64_t linear_smallk_workspace(const rdb_linear_desc *d)
{
    if (!smallk_ok(d)) return 0;
    const int64_t longer = d->in_f > d->out_f ? d->in_f : d->out_f;
    return partial_bytes(d) + cdiv(d->tokens, SK_TT) * cdiv(longer, 256) * 8 + 8 + cdiv(d->tokens, SK_ET) * 8;
}

static bool ws_ok(const rdb_linear_desc *d, const void *ws, int64_t bytes) { return ws && bytes >= linear_smallk_workspace(d) && ((uintptr_t)ws & 7) == 0; }

// Contraction over J (the rows of src) then expansion to `cols` columns: one launch when an expanding block's tags fit one
// wave's lanes (J <= 8192), two otherwise.
template <bool CHASH>
static int contract_expand(float *out, int64_t ld_out, int cols, const float *src, int64_t ld_src, int J, const float *coef, const float *bias,
                           const rdb_linear_desc *d, void *workspace, hipStream_t s)
{
    const int T = (int)d->tokens, k = (int)d->k;
    const int nchunk = (int)cdiv(J, 256), tiles = (int)cdiv(T, SK_TT);
    SkFused f;
    f.c = {(float *)workspace, src, ld_src, coef, T, J, k, d->seed};
    f.e = {out, ld_out, (const float *)workspace, nchunk, coef, bias, T, cols, k, d->seed, nullptr, 0, {nullptr, nullptr, SYNC_SPIN_LIMIT}, nullptr, 0};
    f.slots = reinterpret_cast<unsigned long long *>(static_cast<char *>(workspace) + partial_bytes(d));
    f.c_tiles = tiles;
    f.c_blocks = tiles * nchunk;
    f.e_colblocks = (int)cdiv(cols, 256);
    const int e_blocks = f.e_colblocks * (int)cdiv(T, SK_ET);
    if (nchunk * (SK_ET / SK_TT) <= 64 && one_launch_mode()) {
        f.e.sync = f.slots;
        f.e.sync_tag = next_sync_tag();
        if (int rc = sync_giveups_ptr(&f.e.sync_wait.giveups)) return rc;
        f.counters = reinterpret_cast<unsigned int *>(f.slots + (int64_t)tiles * nchunk) + 2;
        f.e.sync_count = f.counters;
        f.e.sync_consumers = f.e_colblocks;
        smallk_fused_kernel<CHASH><<<f.c_blocks + e_blocks, 256, 0, s>>>(f);
        return check_launch("smallk_fused_kernel");
    }
    smallk_contract_kernel<CHASH><<<dim3((unsigned)tiles, nchunk), 256, 0, s>>>(f.c);
    if (int rc = check_launch("smallk_contract_kernel")) return rc;
    smallk_expand_kernel<!CHASH><<<dim3((unsigned)f.e_colblocks, (unsigned)cdiv(T, SK_ET)), 256, 0, s>>>(f.e);
    return check_launch("smallk_expand_kernel");
}

// Test hook: only the expanding blocks of the one-launch form, waiting (at most `polls` polls each) for a tag that nobody
// publishes.  Every block gives up, fills its share of y with NaN and reports to the give-up counter.
int selftest_giveup_smallk(void *y, int64_t ldy, const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, int polls,
                           hipStream_t s)
{
    if (!smallk_ok(d) || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    const int T = (int)d->tokens, k = (int)d->k, nchunk = (int)cdiv(d->in_f, 256), tiles = (int)cdiv(T, SK_TT);
    if (nchunk * (SK_ET / SK_TT) > 64) return RDB_E_UNSUPPORTED;
    SkExpand e = {(float *)y, ldy, (const float *)workspace, nchunk, (const float *)coef, nullptr, T, (int)d->out_f, k, d->seed, nullptr, 0,
                  {nullptr, nullptr, polls}, nullptr, 0};
    e.sync = reinterpret_cast<unsigned long long *>(static_cast<char *>(workspace) + partial_bytes(d));
    e.sync_tag = next_sync_tag();
    if (int rc = sync_giveups_ptr(&e.sync_wait.giveups)) return rc;
    e.sync_count = reinterpret_cast<unsigned int *>(e.sync + (int64_t)tiles * nchunk) + 2;
    e.sync_consumers = (int)cdiv(d->out_f, 256);
    smallk_expand_kernel<false><<<dim3((unsigned)cdiv(d->out_f, 256), (unsigned)cdiv(T, SK_ET)), 256, 0, s>>>(e);
    return check_launch("smallk_expand_kernel (self-test)");
}

// The three entry points return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
int linear_fwd_smallk(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                      const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    // a layer with a handful of output features (a classifier head) gives the kernel that forms W tiles one column of blocks,
    // each hashing all of N: the factored form wins there whatever the flop counts say (256 -> 10, k = 64, 128 tokens: 19 us
    // against 57)
    const bool few_outputs = d->tokens <= 1024 && d->out_f <= 32;
    if (!smallk_ok(d) || scale_bias || !(smallk_wanted(d) || few_outputs) || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    // z = x . N^T (hashed), y = z . C^T + bias
    return contract_expand<true>((float *)y, ldy, (int)d->out_f, (const float *)x, ldx, (int)d->in_f, (const float *)coef, (const float *)bias, d,
                                 workspace, s);
}

int linear_dx_smallk(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                     void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!smallk_ok(d) || scale_bias || !smallk_wanted(d) || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    // t = dy . C, dx = t . N (hashed)
    return contract_expand<false>((float *)dx, lddx, (int)d->in_f, (const float *)dy, lddy, (int)d->out_f, (const float *)coef, nullptr, d,
                                  workspace, s);
}

// dcoef is overwritten (no zero fill needed).
int linear_dcoef_smallk(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, void *workspace,
                        int64_t workspace_bytes, hipStream_t s)
{
    rdb_linear_desc dd = *d;
    dd.coef_dtype = RDB_F32;  // no coefficients are read here
    if (!smallk_ok(&dd) || !smallk_wanted(&dd) || !ws_ok(&dd, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    const int T = (int)d->tokens, k = (int)d->k;
    float *z = (float *)workspace;
    const int nchunk = (int)cdiv(d->in_f, 256);
    const SkContract c = {z, (const float *)x, ldx, nullptr, T, (int)d->in_f, k, d->seed};
    smallk_contract_kernel<true><<<dim3((unsigned)cdiv(T, SK_TT), nchunk), 256, 0, s>>>(c);
    int rc = check_launch("smallk_contract_kernel<hash>");
    if (rc) return rc;
    dim3 grid((unsigned)cdiv(d->out_f, 256), (unsigned)cdiv(k, 16));
    smallk_dcoef_kernel<<<grid, 256, 0, s>>>(dcoef, (const float *)dy, lddy, z, nchunk, T, (int)d->out_f, k);
    return check_launch("smallk_dcoef_kernel");
}

}  // namespace rdb
