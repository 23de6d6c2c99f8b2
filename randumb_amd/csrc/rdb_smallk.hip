// Fused linear layer, matrix-coef, few tokens (the GEMV-like regime): factored algorithm on the vector ALU, in fp32 whatever the
// dtype of the operands (fp32, or bf16 activations and coefficients).  Two ranges: k <= 64 with up to 1024 tokens (fp32), and
// k <= 256 with up to 96 tokens (both dtypes; 64 for the coefficient gradient), where the matrix-core kernels would run a handful of blocks, each alone with a
// long contraction.
//
// With a handful of tokens the layer moves almost no data (x, C, y) and does almost no arithmetic once W = C . N
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
constexpr int SK_MAX_K = 64;      // the range with many tokens
constexpr int SK_BIG_K = 256;     // the range with few tokens
constexpr int SK_FEW_TOKENS = 96;         // forward and input gradient
constexpr int SK_FEW_TOKENS_DCOEF = 64;   // coefficient gradient (its second kernel walks the tokens one by one)

// out[t, m] = sum_j src[t, j] * B(j, m),  B(j, m) = noise(PRIME*j + m) (HASH) or coef[j, m]; j runs over J = in_f or out_f.
// Block = 8 tokens x one chunk of 256 values of j (blockIdx.y), so that even a single token spreads the hash over many
// compute units; thread = (m % 16, one of 16 interleaved slices of the chunk); the source rows go through LDS (coalesced
// loads, broadcast reads); slices meet in LDS in slice order.  The block writes a partial result, out[chunk][t][m]; the
// expanding kernel adds the chunks up in chunk order while it loads them.
struct SkContract {
    float *out;          // [chunks][T][k] partial sums
    const void *src;     // [T x J], leading dimension ld_src (elements of the kernel's type E)
    int64_t ld_src;
    const void *coef;    // [J x k] (not HASH; E)
    int T, J, k;
    uint32_t seed;
};

// bx: token tile, by: chunk of 256 values of j.  The partial sums are stored at device scope: blocks of the same launch on
// another die may be the ones that read them (smallk_fused_kernel).
// MB: coefficients per block (m0 .. m0 + MB - 1; accumulators per thread: MB / 16 x 8 tokens): 64 where k <= 64, 32 where the
// grid's z spreads a larger k over more blocks; E: float or bf16_t.
template <int MB, typename E, bool HASH> __device__ __forceinline__ void smallk_contract_block(const SkContract &p, int bx, int by, int m0)
{
    constexpr int JC = 256, MC = MB / 16;
    __shared__ float xs[SK_TT][JC];
    __shared__ float red[16][SK_TT][16];
    float *__restrict__ out = p.out;
    const E *__restrict__ src = static_cast<const E *>(p.src);
    const E *__restrict__ coef = static_cast<const E *>(p.coef);
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
        for (int tt = 0; tt < SK_TT; ++tt) xs[tt][tid] = (t0 + tt < T && jc + tid < J) ? elem<E>::load(src + (int64_t)(t0 + tt) * lds_src + jc + tid) : 0.0f;
        __syncthreads();
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            const int m = m0 + c * 16 + m16;
            if (m0 + c * 16 < k) {  // uniform
                uint32_t first = sq5_first((uint32_t)(jc + slice), (uint32_t)m, seed);
                for (int jj = 0; jj < JC / 16; ++jj, first += 16u * PN1) {
                    const int j = jc + slice + 16 * jj;
                    // no branches in here: out-of-range (j, m) read a valid address and are zeroed by a select
                    float b = HASH ? sq5_unit(sq5_tail(first)) : elem<E>::load(coef + (int64_t)(j < J ? j : J - 1) * k + (m < k ? m : k - 1));
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
        if (m0 + c * 16 >= k) break;
#pragma unroll
        for (int tt = 0; tt < SK_TT; ++tt) red[slice][tt][m16] = acc[c][tt];
        __syncthreads();
        if (tid < SK_TT * 16) {
            const int tt = tid >> 4, m = m0 + c * 16 + m16;
            float s = 0.0f;
#pragma unroll
            for (int sl = 0; sl < 16; ++sl) s += red[sl][tt][m16];
            if (t0 + tt < T && m < k) __hip_atomic_store(out + ((int64_t)by * T + t0 + tt) * k + m, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    }
}

template <int MB, typename E, bool HASH> __global__ __launch_bounds__(256) void smallk_contract_kernel(SkContract p)
{
    smallk_contract_block<MB, E, HASH>(p, blockIdx.x, blockIdx.y, blockIdx.z * MB);
}

// out[t, c] = sum_m src[t, m] * B(c, m) (+ bias[c]),  B(c, m) = noise(PRIME*c + m) (HASH) or coef[c, m]; c runs over the
// cols = in_f or out_f.  Block = 256 columns x 16 tokens; a thread owns one column and keeps its 16 B values in registers.
// src holds `nchunk` partial matrices [T x k] (from the contracting kernel), added up here in chunk order.
struct SkExpand {
    void *out;           // [T x cols], leading dimension ld_out (E)
    int64_t ld_out;
    const float *src;    // [nchunk][T][k] partial sums
    int nchunk;
    const void *coef;    // [cols x k] (not HASH; E)
    const void *bias;    // [cols] or NULL (E)
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
template <int KMAX, typename E, bool HASH> __device__ __forceinline__ void smallk_expand_block(const SkExpand &p, int bx, int by)
{
    __shared__ __align__(16) float s[SK_ET][KMAX];
    E *__restrict__ out = static_cast<E *>(p.out);
    const float *__restrict__ src = p.src;
    const E *__restrict__ coef = static_cast<const E *>(p.coef);
    const E *__restrict__ bias = static_cast<const E *>(p.bias);
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
            const float v = HASH ? sq5_unit(sq5_tail(sq5_first((uint32_t)cc, (uint32_t)m, seed))) : elem<E>::load(coef + (int64_t)cc * k + ((m < k) ? m : k - 1));
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
                    if (t0 + tt < T) elem<E>::store(out + (int64_t)(t0 + tt) * ld_out + c, __uint_as_float(0x7fc00000u));
            return;
        }
    }
    // s = sum of the partial matrices in chunk order; columns from k on take part as zeros.  A thread owns up to 4 entries
    // and keeps the loads of 8 chunks of all of them in flight at once: the kernel is a chain of memory latencies otherwise.
    {
        // entry i of a thread: token (tid / KMAX) + (256 / KMAX) i, coefficient tid % KMAX (no division by k)
        constexpr int PER = SK_ET * KMAX / 256, CB = 8, TSTEP = 256 / KMAX;
        static_assert(256 % KMAX == 0 && SK_ET % TSTEP == 0, "the tile's entries split evenly over the threads");
        const int em = tid % KMAX, et = tid / KMAX;
        float v[PER];
        const float *ptr[PER];
        bool ok[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int tt = et + TSTEP * i;
            v[i] = 0.0f;
            ok[i] = em < k && t0 + tt < T;
            ptr[i] = ok[i] ? src + (int64_t)(t0 + tt) * k + em : src;   // always a valid address
        }
        const int64_t stride = (int64_t)T * k;
        for (int c0 = 0; c0 < nchunk; c0 += CB) {
            float l[PER][CB];
#pragma unroll
            for (int i = 0; i < PER; ++i)
#pragma unroll
                for (int u = 0; u < CB; ++u)   // device scope: possibly written by another die during this launch
                    l[i][u] = __hip_atomic_load(ptr[i] + (int64_t)((c0 + u < nchunk) ? c0 + u : nchunk - 1) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int i = 0; i < PER; ++i)
#pragma unroll
                for (int u = 0; u < CB; ++u) v[i] += (ok[i] && c0 + u < nchunk) ? l[i][u] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) s[et + TSTEP * i][em] = ok[i] ? v[i] : 0.0f;   // every entry of s is somebody's
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
                                     : elem<E>::load(coef + (int64_t)c * k + ((mc + m < k) ? mc + m : k - 1));
                b[m] = (mc + m < k) ? v : 0.0f;
            }
        }
        // mc <= KMAX - 16 and m <= 15: always inside the KMAX columns of s
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
    const float bv = bias ? elem<E>::load(bias + c) : 0.0f;
#pragma unroll
    for (int tt = 0; tt < SK_ET; ++tt)
        if (t0 + tt < T) elem<E>::store(out + (int64_t)(t0 + tt) * ld_out + c, acc[tt] + bv);
}

template <int KMAX, typename E, bool HASH> __global__ __launch_bounds__(256) void smallk_expand_kernel(SkExpand p)
{
    smallk_expand_block<KMAX, E, HASH>(p, blockIdx.x, blockIdx.y);
}

// zsum[e] = part[0][e] + part[1][e] + ... in chunk order, one entry [token, coefficient] per thread: k beyond 64, where many
// expanding blocks share a token's partial matrices and each of them adding them up again costs more than this launch
__global__ __launch_bounds__(256) void smallk_sum_chunks_kernel(float *__restrict__ zsum, const float *__restrict__ part, int64_t n, int nchunk)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n) return;
    float v = 0.0f;
    for (int c0 = 0; c0 < nchunk; c0 += 16) {
        float l[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) l[u] = part[(int64_t)((c0 + u < nchunk) ? c0 + u : nchunk - 1) * n + e];
#pragma unroll
        for (int u = 0; u < 16; ++u) v += (c0 + u < nchunk) ? l[u] : 0.0f;
    }
    zsum[e] = v;
}

// The same for k up to 256 and few tokens, where one thread per column would leave the chip empty and every thread alone with
// k values of B: block = 32 columns x 16 tokens, thread = (column, one of eight ranges of 32 coefficients); the ranges of a
// column meet in LDS in range order.  The block's rows of C pass through LDS (read from memory along the rows, by the threads
// along the columns).  A launch of its own, after the contracting kernel's and smallk_sum_chunks_kernel's (src = the sum,
// nchunk = 1).
constexpr int SKW_COLS = 32, SKW_RANGES = 8;
template <typename E, bool HASH> __global__ __launch_bounds__(256) void smallk_expand_wide_kernel(SkExpand p)
{
    constexpr int KW = SK_BIG_K, RANGE = KW / SKW_RANGES, CLD = KW + 1;
    static_assert(SKW_COLS * SKW_RANGES == 256 && SK_ET % SKW_RANGES == 0 && RANGE % 16 == 0, "thread layout of the wide expansion");
    __shared__ __align__(16) float s[SK_ET][KW];
    __shared__ float cs[SKW_COLS * CLD];   // C rows, stride CLD (conflict-free down a column); later the ranges' sums [range][token][column]
    static_assert(SKW_RANGES * SK_ET * SKW_COLS <= SKW_COLS * CLD, "the ranges' sums fit where the C rows were");
    E *__restrict__ out = static_cast<E *>(p.out);
    const float *__restrict__ src = p.src;
    const E *__restrict__ coef = static_cast<const E *>(p.coef);
    const E *__restrict__ bias = static_cast<const E *>(p.bias);
    const int64_t ld_out = p.ld_out;
    const int nchunk = p.nchunk, T = p.T, cols = p.cols, k = p.k;
    const uint32_t seed = p.seed;
    const int tid = threadIdx.x, col = tid % SKW_COLS, g = tid / SKW_COLS;
    const int c0 = blockIdx.x * SKW_COLS, c = c0 + col, t0 = blockIdx.y * SK_ET;
    const int cc = c < cols ? c : cols - 1;
    if (!HASH) {
        // the block's rows of C: a wave reads 64 consecutive values of one row at a time; all of a thread's 32 loads are in
        // flight before the first is stored (rows past cols and coefficients past k: zeros)
        const int r0 = tid >> 6, m0 = tid & 63;
        float cv[SKW_COLS / 4][KW / 64];
#pragma unroll
        for (int r = 0; r < SKW_COLS / 4; ++r)
#pragma unroll
            for (int j = 0; j < KW / 64; ++j) {
                const int row = r0 + 4 * r, m = m0 + 64 * j;
                const bool in = c0 + row < cols && m < k;   // (a valid address either way; the select makes the zero)
                const float x = elem<E>::load(coef + (int64_t)(c0 + row < cols ? c0 + row : cols - 1) * k + (m < k ? m : k - 1));
                cv[r][j] = in ? x : 0.0f;
            }
#pragma unroll
        for (int r = 0; r < SKW_COLS / 4; ++r)
#pragma unroll
            for (int j = 0; j < KW / 64; ++j) cs[(r0 + 4 * r) * CLD + m0 + 64 * j] = cv[r][j];
    }
    // s = sum of the partial matrices in chunk order (as a rule one: smallk_sum_chunks_kernel ran first); thread = coefficient,
    // one entry per token; coefficients from k on and tokens past the end take part as zeros
    {
        static_assert(KW == 256, "one coefficient per thread");
        constexpr int CB = 4;
        // no branches around the loads: an entry that does not exist reads a valid address and becomes 0 by a select
        const int m = tid < k ? tid : k - 1;
        float v[SK_ET];
        const float *ptr[SK_ET];
        const int64_t stride = (int64_t)T * k;
#pragma unroll
        for (int i = 0; i < SK_ET; ++i) {
            v[i] = 0.0f;
            ptr[i] = src + (int64_t)(t0 + i < T ? t0 + i : T - 1) * k + m;
        }
        if (nchunk == 1) {
#pragma unroll
            for (int i = 0; i < SK_ET; ++i) v[i] = ptr[i][0];
        } else {
            for (int q0 = 0; q0 < nchunk; q0 += CB) {
                float l[SK_ET][CB];
#pragma unroll
                for (int i = 0; i < SK_ET; ++i)
#pragma unroll
                    for (int u = 0; u < CB; ++u) l[i][u] = ptr[i][(int64_t)((q0 + u < nchunk) ? q0 + u : nchunk - 1) * stride];
#pragma unroll
                for (int i = 0; i < SK_ET; ++i)
#pragma unroll
                    for (int u = 0; u < CB; ++u) v[i] += (q0 + u < nchunk) ? l[i][u] : 0.0f;
            }
        }
#pragma unroll
        for (int i = 0; i < SK_ET; ++i) s[i][tid] = (tid < k && t0 + i < T) ? v[i] : 0.0f;
    }
    __syncthreads();
    float acc[SK_ET];
#pragma unroll
    for (int tt = 0; tt < SK_ET; ++tt) acc[tt] = 0.0f;
    const float *crow = cs + (c < cols ? col : 0) * CLD;
    for (int mc = g * RANGE; mc < (g + 1) * RANGE && mc < k; mc += 16) {
        float b[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) {   // branch-free: a coefficient from k on reads a valid address and becomes 0
            const float v = HASH ? sq5_unit(sq5_tail(sq5_first((uint32_t)cc, (uint32_t)(mc + m), seed))) : crow[mc + m];   // zeros from k on
            b[m] = (mc + m < k) ? v : 0.0f;
        }
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
    __syncthreads();   // everybody is done with the C rows
    float *red = cs;
#pragma unroll
    for (int tt = 0; tt < SK_ET; ++tt) red[(g * SK_ET + tt) * SKW_COLS + col] = acc[tt];
    __syncthreads();
    if (c >= cols) return;
    const float bv = bias ? elem<E>::load(bias + c) : 0.0f;
#pragma unroll
    for (int q = 0; q < SK_ET / SKW_RANGES; ++q) {   // this thread finishes two of the column's tokens
        const int tt = g * (SK_ET / SKW_RANGES) + q;
        float v = red[tt * SKW_COLS + col];
#pragma unroll
        for (int r = 1; r < SKW_RANGES; ++r) v += red[(r * SK_ET + tt) * SKW_COLS + col];
        if (t0 + tt < T) elem<E>::store(out + (int64_t)(t0 + tt) * ld_out + c, v + bv);
    }
}

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

template <int KMAX, typename E, bool CHASH> __global__ __launch_bounds__(256) void smallk_fused_kernel(SkFused p)
{
    const int b = blockIdx.x;
    if (b < p.c_blocks) {
        const int bx = b % p.c_tiles, by = b / p.c_tiles;
        // a replayed launch carries the tag it was recorded with: should a consumer of an earlier replay have given up, the slot
        // may still hold it (the consumers clear the slots only when all of them got past their wait)
        if (threadIdx.x == 0) __hip_atomic_store(p.slots + (int64_t)bx * p.e.nchunk + by, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        smallk_contract_block<KMAX, E, CHASH>(p.c, bx, by, 0);
        if (by == 0 && bx % (SK_ET / SK_TT) == 0 && threadIdx.x == 0)
            __hip_atomic_store(p.counters + bx / (SK_ET / SK_TT), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        publish_tag(p.slots + (int64_t)bx * p.e.nchunk + by, p.e.sync_tag);
    } else {
        const int e = b - p.c_blocks;
        smallk_expand_block<KMAX, E, !CHASH>(p.e, e % p.e_colblocks, e / p.e_colblocks);
    }
}

// dC[o, m] = sum_t dy[t, o] * z[t, m].  Block = 256 output rows x one chunk of 16 coefficients; z goes through LDS in tiles
// of 64 tokens; a thread owns one output row and walks the tokens in order.
template <typename E>
__global__ __launch_bounds__(256) void smallk_dcoef_kernel(float *__restrict__ dcoef, const E *__restrict__ dy, int64_t lddy,
                                                           const float *__restrict__ z, int nchunk, int T, int out_f, int k)
{
    __shared__ __align__(16) float zs[64][16];
    const int tid = threadIdx.x;
    const int o = blockIdx.x * 256 + tid, mc = blockIdx.y * 16;
    float acc[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] = 0.0f;
    for (int t0 = 0; t0 < T; t0 += 64) {
        {   // a thread's four entries of the z tile, the loads of eight chunks of all four in flight together (an entry that does
            // not exist reads a valid address and becomes 0 by a select)
            const float *at[4];
            float zv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int e = tid + 256 * q, tt = e >> 4, m = e & 15;
                at[q] = z + (int64_t)(t0 + tt < T ? t0 + tt : T - 1) * k + (mc + m < k ? mc + m : k - 1);
                zv[q] = 0.0f;
            }
            const int64_t stride = (int64_t)T * k;
            for (int c0 = 0; c0 < nchunk; c0 += 8) {
                float l[4][8];
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int u = 0; u < 8; ++u) l[q][u] = at[q][(int64_t)((c0 + u < nchunk) ? c0 + u : nchunk - 1) * stride];
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int u = 0; u < 8; ++u) zv[q] += (c0 + u < nchunk) ? l[q][u] : 0.0f;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int e = tid + 256 * q, tt = e >> 4, m = e & 15;
                zs[tt][m] = (t0 + tt < T && mc + m < k) ? zv[q] : 0.0f;
            }
        }
        __syncthreads();
        if (o < out_f) {
            const int n = (T - t0 < 64) ? T - t0 : 64;
            for (int tt = 0; tt < n; ++tt) {
                const float g = elem<E>::load(dy + (int64_t)(t0 + tt) * lddy + o);
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
// The regimes this file is for; AUTO additionally wants the factored form to be the cheaper way.
static bool smallk_ok(const rdb_linear_desc *d)
{
    const bool f32 = d->act_dtype == RDB_F32 && d->coef_dtype == RDB_F32, b16 = d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16;
    if (!(f32 || b16) || d->coef_rows == 0 || d->k <= 0 || d->tokens <= 0 || d->in_f <= 0 || d->out_f <= 0 || d->in_f >= (1 << 30) ||
        d->out_f >= (1 << 30))
        return false;
    if (f32 && d->k <= SK_MAX_K && d->tokens <= 4096) return true;
    return d->k <= SK_BIG_K && d->tokens <= SK_FEW_TOKENS;
}
enum SkDirection { SK_FWD, SK_DX, SK_DCOEF };
static bool smallk_wanted(const rdb_linear_desc *d, int dir)
{
    const bool cheaper = d->k * (d->in_f + d->out_f) < d->in_f * d->out_f;
    if (d->act_dtype == RDB_F32 && d->k <= SK_MAX_K) return d->algo == RDB_ALGO_FACTORED || (d->tokens <= 1024 && cheaper);
    if (d->tokens > (dir == SK_DCOEF ? SK_FEW_TOKENS_DCOEF : SK_FEW_TOKENS) || !cheaper) return false;
    if (d->k <= SK_MAX_K) return true;
    // k beyond 64 (contraction over J: in_f for the forward and the coefficient gradient's z, out_f for the input gradient): in
    // bf16 the matrix-core kernels' time grows with the contraction (a few blocks, each alone with all of it): below about
    // 1536 values they are ahead (768 -> 3072, 16 tokens: forward 15 us against 16, coefficient gradient 17 against 17-24),
    // beyond it behind (4096 -> 4096: 39 against 16, 41 against 18)
    const int64_t J = dir == SK_DX ? d->out_f : d->in_f;
    return d->act_dtype == RDB_F32 || J >= 1536;
}

// scratch: one partial [tokens x k] fp32 matrix per 256-chunk of the longer of in_f and out_f, then the tag slots of the
// one-launch form (one per token tile and chunk), 8 bytes not in use and a counter per 16 tokens (a waiting block that gives
// up reports to the library's per-device counter: the scratch may be the caller's and gone by the time anybody looks)
static int64_t partial_bytes(const rdb_linear_desc *d)
{
    const int64_t longer = d->in_f > d->out_f ? d->in_f : d->out_f;
    return (cdiv(longer, 256) * d->tokens * d->k * (int64_t)sizeof(float) + 7) / 8 * 8;
}
// k beyond 64: behind the partial matrices their sum [tokens x k]
static int64_t zsum_bytes(const rdb_linear_desc *d) { return (d->tokens * d->k * (int64_t)sizeof(float) + 7) / 8 * 8; }
int64_t linear_smallk_workspace(const rdb_linear_desc *d)
{
    if (!smallk_ok(d)) return 0;
    if (d->k > SK_MAX_K) return partial_bytes(d) + zsum_bytes(d);
    const int64_t longer = d->in_f > d->out_f ? d->in_f : d->out_f;
    return partial_bytes(d) + cdiv(d->tokens, SK_TT) * cdiv(longer, 256) * 8 + 8 + cdiv(d->tokens, SK_ET) * 8;
}

static bool ws_ok(const rdb_linear_desc *d, const void *ws, int64_t bytes) { return ws && bytes >= linear_smallk_workspace(d) && ((uintptr_t)ws & 7) == 0; }

// Contraction over J (the rows of src) then expansion to `cols` columns: one launch when an expanding block's tags fit one
// wave's lanes (J <= 8192), two otherwise.
template <int KMAX, typename E, bool CHASH>
static int contract_expand_as(void *out, int64_t ld_out, int cols, const void *src, int64_t ld_src, int J, const void *coef, const void *bias,
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
        smallk_fused_kernel<KMAX, E, CHASH><<<f.c_blocks + e_blocks, 256, 0, s>>>(f);
        return check_launch("smallk_fused_kernel");
    }
    smallk_contract_kernel<KMAX, E, CHASH><<<dim3((unsigned)tiles, nchunk), 256, 0, s>>>(f.c);
    if (int rc = check_launch("smallk_contract_kernel")) return rc;
    smallk_expand_kernel<KMAX, E, !CHASH><<<dim3((unsigned)f.e_colblocks, (unsigned)cdiv(T, SK_ET)), 256, 0, s>>>(f.e);
    return check_launch("smallk_expand_kernel");
}
// the instance for the request's k and dtype (activations and coefficients have the same one: smallk_ok)
// k beyond 64 (few tokens): the contraction spread over the grid's z in ranges of SK_MB coefficients, the sum of its chunks,
// then the wide expansion; three launches
constexpr int SK_MB = 32;
static int sum_chunks(float *zsum, const float *part, const rdb_linear_desc *d, int nchunk, hipStream_t s)
{
    const int64_t n = d->tokens * d->k;
    smallk_sum_chunks_kernel<<<(unsigned)cdiv(n, 256), 256, 0, s>>>(zsum, part, n, nchunk);
    return check_launch("smallk_sum_chunks_kernel");
}
template <typename E, bool CHASH>
static int contract_expand_wide(void *out, int64_t ld_out, int cols, const void *src, int64_t ld_src, int J, const void *coef, const void *bias,
                                const rdb_linear_desc *d, void *workspace, hipStream_t s)
{
    const int T = (int)d->tokens, k = (int)d->k, nchunk = (int)cdiv(J, 256);
    if (nchunk > 65535) return RDB_E_UNSUPPORTED;   // the grid's y
    const SkContract c = {(float *)workspace, src, ld_src, coef, T, J, k, d->seed};
    float *zsum = reinterpret_cast<float *>(static_cast<char *>(workspace) + partial_bytes(d));
    const SkExpand e = {out, ld_out, zsum, 1, coef, bias, T, cols, k, d->seed, nullptr, 0, {nullptr, nullptr, 0}, nullptr, 0};
    smallk_contract_kernel<SK_MB, E, CHASH><<<dim3((unsigned)cdiv(T, SK_TT), nchunk, (unsigned)cdiv(k, SK_MB)), 256, 0, s>>>(c);
    if (int rc = check_launch("smallk_contract_kernel")) return rc;
    if (int rc = sum_chunks(zsum, (const float *)workspace, d, nchunk, s)) return rc;
    smallk_expand_wide_kernel<E, !CHASH><<<dim3((unsigned)cdiv(cols, SKW_COLS), (unsigned)cdiv(T, SK_ET)), 256, 0, s>>>(e);
    return check_launch("smallk_expand_wide_kernel");
}
template <bool CHASH>
static int contract_expand(void *out, int64_t ld_out, int cols, const void *src, int64_t ld_src, int J, const void *coef, const void *bias,
                           const rdb_linear_desc *d, void *workspace, hipStream_t s)
{
    const bool b16 = d->act_dtype == RDB_BF16;
    if (d->k <= SK_MAX_K)
        return b16 ? contract_expand_as<SK_MAX_K, bf16_t, CHASH>(out, ld_out, cols, src, ld_src, J, coef, bias, d, workspace, s)
                   : contract_expand_as<SK_MAX_K, float, CHASH>(out, ld_out, cols, src, ld_src, J, coef, bias, d, workspace, s);
    return b16 ? contract_expand_wide<bf16_t, CHASH>(out, ld_out, cols, src, ld_src, J, coef, bias, d, workspace, s)
               : contract_expand_wide<float, CHASH>(out, ld_out, cols, src, ld_src, J, coef, bias, d, workspace, s);
}

// Test hook: only the expanding blocks of the one-launch form, waiting (at most `polls` polls each) for a tag that nobody
// publishes.  Every block gives up, fills its share of y with NaN and reports to the give-up counter.
int selftest_giveup_smallk(void *y, int64_t ldy, const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, int polls,
                           hipStream_t s)
{
    if (!smallk_ok(d) || d->act_dtype != RDB_F32 || d->k > SK_MAX_K || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    const int T = (int)d->tokens, k = (int)d->k, nchunk = (int)cdiv(d->in_f, 256), tiles = (int)cdiv(T, SK_TT);
    if (nchunk * (SK_ET / SK_TT) > 64) return RDB_E_UNSUPPORTED;
    SkExpand e = {y, ldy, (const float *)workspace, nchunk, coef, nullptr, T, (int)d->out_f, k, d->seed, nullptr, 0,
                  {nullptr, nullptr, polls}, nullptr, 0};
    e.sync = reinterpret_cast<unsigned long long *>(static_cast<char *>(workspace) + partial_bytes(d));
    e.sync_tag = next_sync_tag();
    if (int rc = sync_giveups_ptr(&e.sync_wait.giveups)) return rc;
    e.sync_count = reinterpret_cast<unsigned int *>(e.sync + (int64_t)tiles * nchunk) + 2;
    e.sync_consumers = (int)cdiv(d->out_f, 256);
    smallk_expand_kernel<SK_MAX_K, float, false><<<dim3((unsigned)cdiv(d->out_f, 256), (unsigned)cdiv(T, SK_ET)), 256, 0, s>>>(e);
    return check_launch("smallk_expand_kernel (self-test)");
}

// The three entry points return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
int linear_fwd_smallk(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                      const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    // a layer with a handful of output features (a classifier head) gives the kernel that forms W tiles one column of blocks,
    // each hashing all of N: the factored form wins there whatever the flop counts say (256 -> 10, k = 64, 128 tokens: 19 us
    // against 57)
    const bool few_outputs = d->act_dtype == RDB_F32 && d->k <= SK_MAX_K && d->tokens <= 1024 && d->out_f <= 32;
    if (!smallk_ok(d) || scale_bias || !(smallk_wanted(d, SK_FWD) || few_outputs) || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    // z = x . N^T (hashed), y = z . C^T + bias
    return contract_expand<true>(y, ldy, (int)d->out_f, x, ldx, (int)d->in_f, coef, bias, d, workspace, s);
}

int linear_dx_smallk(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                     void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!smallk_ok(d) || scale_bias || !smallk_wanted(d, SK_DX) || !ws_ok(d, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    // t = dy . C, dx = t . N (hashed)
    return contract_expand<false>(dx, lddx, (int)d->in_f, dy, lddy, (int)d->out_f, coef, nullptr, d, workspace, s);
}

// dcoef is overwritten (no zero fill needed).
int linear_dcoef_smallk(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, void *workspace,
                        int64_t workspace_bytes, hipStream_t s)
{
    rdb_linear_desc dd = *d;
    dd.coef_dtype = d->act_dtype;  // no coefficients are read here
    if (!smallk_ok(&dd) || !smallk_wanted(&dd, SK_DCOEF) || !ws_ok(&dd, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    const int T = (int)d->tokens, k = (int)d->k;
    const bool b16 = d->act_dtype == RDB_BF16;
    float *z = (float *)workspace;
    const int nchunk = (int)cdiv(d->in_f, 256);
    const SkContract c = {z, x, ldx, nullptr, T, (int)d->in_f, k, d->seed};
    const dim3 cgrid((unsigned)cdiv(T, SK_TT), nchunk);
    if (k <= SK_MAX_K) {
        if (b16) smallk_contract_kernel<SK_MAX_K, bf16_t, true><<<cgrid, 256, 0, s>>>(c);
        else smallk_contract_kernel<SK_MAX_K, float, true><<<cgrid, 256, 0, s>>>(c);
    } else {
        const dim3 wgrid(cgrid.x, cgrid.y, (unsigned)cdiv(k, SK_MB));
        if (b16) smallk_contract_kernel<SK_MB, bf16_t, true><<<wgrid, 256, 0, s>>>(c);
        else smallk_contract_kernel<SK_MB, float, true><<<wgrid, 256, 0, s>>>(c);
    }
    int rc = check_launch("smallk_contract_kernel<hash>");
    if (rc) return rc;
    const float *zz = z;
    int zchunks = nchunk;
    if (k > SK_MAX_K) {   // every block of the kernel below would add the chunks up again
        float *zsum = reinterpret_cast<float *>(static_cast<char *>(workspace) + partial_bytes(&dd));
        if ((rc = sum_chunks(zsum, z, &dd, nchunk, s))) return rc;
        zz = zsum;
        zchunks = 1;
    }
    dim3 grid((unsigned)cdiv(d->out_f, 256), (unsigned)cdiv(k, 16));
    if (b16) smallk_dcoef_kernel<bf16_t><<<grid, 256, 0, s>>>(dcoef, (const bf16_t *)dy, lddy, zz, zchunks, T, (int)d->out_f, k);
    else smallk_dcoef_kernel<float><<<grid, 256, 0, s>>>(dcoef, (const float *)dy, lddy, zz, zchunks, T, (int)d->out_f, k);
    return check_launch("smallk_dcoef_kernel");
}

}  // namespace rdb
