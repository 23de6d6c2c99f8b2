// Fused linear layer on a vector-coef pseudorandom weight (the reference's form: one coefficient vector c[k] for the whole
// tensor, W_flat[a] = sum_m noise(PRIME*a + m) * c[m], src/rten_cpp/RandumbTensor.py:235-290), forward and input gradient,
// for up to a few thousand tokens.
//
// Every weight element costs k hashes, so regenerating W is the whole cost (604 M hashes at 768 x 3072, k = 256) and what
// matters is that all of the chip's vector ALUs share it.  A kernel that gives a block one tile of the OUTPUT has only
// out_f / 128 x tokens / 128 blocks, each hashing a whole strip of W (24 blocks at 128 tokens).  Here a block owns a tile of W
// instead, 64 columns of the output x 32 values of the contraction: it forms the tile once (8 elements a thread, k hashes each,
// one rounding to the activations' dtype, as materialize().to(dtype) does, RandumbTensor.py:892), keeps it in LDS and streams
// all tokens through it on the matrix cores; the products of the contraction's chunks are partial outputs [chunk][tokens x
// columns] in fp32 in the caller's workspace, added up in chunk order by a second kernel (no atomics: the same bits from run to
// run).  W is never written to memory.  One kernel serves both products:
//   forward  y[t, o]  = sum_i x[t, i]  * W[o, i]    columns = output features, contraction = input features
//   dx       dx[t, i] = sum_o dy[t, o] * W[o, i]    columns = input features,  contraction = output features
// Replaces materialize() + dense product (RandumbTensor.py:942-952) and MmBackward on the re-materialised weight.
#include <algorithm>

#include "rdb_tile.hpp"

namespace rdb {

constexpr int VS_BC = 64, VS_BJ = 32, VS_BT = 128, VS_COEF_CHUNK = 2048;

struct VsParams {
    const void *src;          // [tokens x J], leading dimension ld_src
    int64_t ld_src;
    const void *coef;         // [k], coef_dtype
    const void *scale_bias;   // NULL or one value of coef_dtype: W += s * noise(a)
    float *partial;           // [chunks][tokens][C]
    int tokens, C, J, k;
    int64_t sC, sJ;           // storage offset of the element at (column c, contraction value j): c * sC + j * sJ
    uint32_t seed;
    int coef_dtype;
    int tiles_c, chunks;
    int vec_src;              // 16-byte loads of src allowed
};

template <typename T> __global__ __launch_bounds__(TILE_THREADS, 2) void vecsplit_kernel(VsParams p)
{
    constexpr int LD = VS_BJ + MMA<T>::PAD;
    __shared__ __align__(16) T Ws[VS_BC * LD];    // Ws[c][j]: the "B" operand
    __shared__ __align__(16) T As[VS_BT * LD];    // As[tok][j]
    __shared__ float cs[VS_COEF_CHUNK];
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5;
    const float sb = p.scale_bias ? load_as_f32(p.scale_bias, p.coef_dtype, 0) : 0.0f;
    const int items = p.tiles_c * p.chunks;
    for (int item = blockIdx.x; item < items; item += gridDim.x) {
        // chunk fastest: the blocks running at one time read the same token rows of src
        const int chunk = item % p.chunks, ct = item / p.chunks, c0 = ct * VS_BC, j0 = chunk * VS_BJ;
        // ---- the tile of W: thread t owns elements lin = e * 256 + t, column lin / 32, contraction value lin % 32
        constexpr int PER = VS_BC * VS_BJ / TILE_THREADS;
        uint32_t first[PER], addr[PER];
        float acc[PER];
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int lin = e * TILE_THREADS + t;
            addr[e] = (uint32_t)((int64_t)(c0 + lin / VS_BJ) * p.sC + (int64_t)(j0 + lin % VS_BJ) * p.sJ);
            first[e] = addr[e] * PN1 + p.seed;   // first-round value for m = 0; + N1 per step of m
            acc[e] = 0.0f;
        }
        for (int m0 = 0; m0 < p.k; m0 += VS_COEF_CHUNK) {
            const int cnt = p.k - m0 < VS_COEF_CHUNK ? p.k - m0 : VS_COEF_CHUNK;
            __syncthreads();   // the previous chunk of coefficients (and the previous item's tiles) are no longer read
            for (int j = t; j < cnt; j += TILE_THREADS) cs[j] = load_as_f32(p.coef, p.coef_dtype, m0 + j);
            __syncthreads();
#pragma unroll 2
            for (int j = 0; j < cnt; ++j) {
                const float c = cs[j];
#pragma unroll
                for (int e = 0; e < PER; ++e) {
                    acc[e] = fmaf(sq5_unit(sq5_tail(first[e])), c, acc[e]);
                    first[e] += SQ5_N1;
                }
            }
        }
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int lin = e * TILE_THREADS + t, cc = lin / VS_BJ, jj = lin % VS_BJ;
            float v = acc[e];
            if (p.scale_bias) v += sb * noise1d(addr[e], p.seed);
            // columns and contraction values past the end: exact zeros, whatever the hash says there
            Ws[cc * LD + jj] = (c0 + cc < p.C && j0 + jj < p.J) ? from_f32<T>(v) : from_f32<T>(0.0f);
        }
        // ---- all tokens through it
        float *out = p.partial + (int64_t)chunk * p.tokens * p.C;
        for (int tok0 = 0; tok0 < p.tokens; tok0 += VS_BT) {
            __syncthreads();   // Ws complete; As free
            load_tile_rowmajor<T, VS_BT, VS_BJ>(As, LD, (const T *)p.src, p.ld_src, tok0, p.tokens, j0, p.J, p.vec_src != 0);
            __syncthreads();
            f32x16 d[2] = {zero16(), zero16()};
#pragma unroll
            for (int ks = 0; ks < VS_BJ / 16; ++ks) {
                const typename MMA<T>::Frag fa = MMA<T>::load(As + (wave * 32 + r) * LD + ks * 16 + g * 8);
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) MMA<T>::mma(d[ni], fa, MMA<T>::load(Ws + (ni * 32 + r) * LD + ks * 16 + g * 8));
            }
            // d[ni][j]: token tok0 + 32 wave + 8 (j / 4) + 4 g + j % 4, column c0 + 32 ni + r
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const int c = c0 + ni * 32 + r;
                if (c >= p.C) continue;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int tok = tok0 + wave * 32 + 8 * (j / 4) + 4 * g + (j % 4);
                    if (tok < p.tokens) out[(int64_t)tok * p.C + c] = d[ni][j];
                }
            }
        }
    }
}

// out[t, c] = sum over the chunks, in chunk order, of partial[chunk][t][c] (+ bias[c])
template <typename T>
__global__ __launch_bounds__(256) void vecsplit_sum_kernel(T *__restrict__ out, int64_t ld_out, const float *__restrict__ partial, const T *__restrict__ bias,
                                                           int tokens, int C, int chunks)
{
    const int64_t n = (int64_t)tokens * C;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
        float v = 0.0f;
        for (int c0 = 0; c0 < chunks; c0 += 8) {   // eight loads in flight at a time; the additions stay in chunk order
            float l[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) l[u] = partial[(int64_t)(c0 + u < chunks ? c0 + u : chunks - 1) * n + e];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + u < chunks) v += l[u];
        }
        const int64_t tok = e / C, c = e % C;
        if (bias) v += to_f32<T>(bias[c]);
        out[tok * ld_out + c] = from_f32<T>(v);
    }
}

// ----------------------------------------------------------------------------------------------- host side
constexpr int64_t VS_MAX_TOKENS = 4096, VS_MAX_WORKSPACE = 1ll << 30;

// C: columns of the output, J: contraction length
static int64_t vs_bytes(int64_t tokens, int64_t C, int64_t J) { return cdiv(J, VS_BJ) * tokens * C * (int64_t)sizeof(float); }

static bool vs_ok(const rdb_linear_desc *d)
{
    return d->coef_rows == 0 && (d->act_dtype == RDB_F32 || d->act_dtype == RDB_BF16) && d->tokens > 0 && d->tokens <= VS_MAX_TOKENS && d->in_f > 0 &&
           d->out_f > 0 && d->k > 0 && d->in_f < (1 << 30) && d->out_f < (1 << 30) && d->k < (1 << 30);
}

// scratch of the forward (op 0) or the input gradient (op 1) in this form; 0 when it does not apply
int64_t linear_vecsplit_workspace(int op, const rdb_linear_desc *d)
{
    if (!vs_ok(d)) return 0;
    const int64_t b = op == RDB_OP_LINEAR_FWD ? vs_bytes(d->tokens, d->out_f, d->in_f) : op == RDB_OP_LINEAR_BWD_DX ? vs_bytes(d->tokens, d->in_f, d->out_f) : 0;
    return b <= VS_MAX_WORKSPACE ? b : 0;
}

template <typename T>
static int vs_launch(void *out, int64_t ld_out, int64_t C, const void *src, int64_t ld_src, int64_t J, int64_t sC, int64_t sJ, const void *coef,
                     const void *scale_bias, const void *bias, const rdb_linear_desc *d, int num_cus, void *workspace, hipStream_t s)
{
    VsParams p;
    p.src = src;
    p.ld_src = ld_src;
    p.coef = coef;
    p.scale_bias = scale_bias;
    p.partial = (float *)workspace;
    p.tokens = (int)d->tokens;
    p.C = (int)C;
    p.J = (int)J;
    p.k = (int)d->k;
    p.sC = sC;
    p.sJ = sJ;
    p.seed = d->seed;
    p.coef_dtype = d->coef_dtype;
    p.tiles_c = (int)cdiv(C, VS_BC);
    p.chunks = (int)cdiv(J, VS_BJ);
    p.vec_src = (((uintptr_t)src & 15) == 0 && (ld_src * (int64_t)sizeof(T)) % 16 == 0) ? 1 : 0;
    const int64_t items = (int64_t)p.tiles_c * p.chunks;
    // two blocks per compute unit, each walking the items with the grid's stride: all vector ALUs stay busy to within one item
    const int grid = (int)std::min<int64_t>(items, 2 * (int64_t)num_cus);
    vecsplit_kernel<T><<<grid, TILE_THREADS, 0, s>>>(p);
    if (int rc = check_launch("vecsplit_kernel")) return rc;
    const int64_t n = d->tokens * C;
    vecsplit_sum_kernel<T><<<(unsigned)std::min<int64_t>(cdiv(n, 256), 4096), 256, 0, s>>>((T *)out, ld_out, p.partial, (const T *)bias, p.tokens, p.C, p.chunks);
    return check_launch("vecsplit_sum_kernel");
}

// Return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
int linear_fwd_vecsplit(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                        const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    const int64_t need = linear_vecsplit_workspace(RDB_OP_LINEAR_FWD, d);
    if (need <= 0 || !workspace || workspace_bytes < need || ((uintptr_t)workspace & 15)) return RDB_E_UNSUPPORTED;
    // weight element (o, i) at o * sO + i * sI: columns = o, contraction = i
    if (d->act_dtype == RDB_BF16)
        return vs_launch<bf16_t>(y, ldy, d->out_f, x, ldx, d->in_f, d->sO, d->sI, coef, scale_bias, bias, d, num_cus, workspace, s);
    return vs_launch<float>(y, ldy, d->out_f, x, ldx, d->in_f, d->sO, d->sI, coef, scale_bias, bias, d, num_cus, workspace, s);
}

int linear_dx_vecsplit(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                       int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    const int64_t need = linear_vecsplit_workspace(RDB_OP_LINEAR_BWD_DX, d);
    if (need <= 0 || !workspace || workspace_bytes < need || ((uintptr_t)workspace & 15)) return RDB_E_UNSUPPORTED;
    // columns = i, contraction = o
    if (d->act_dtype == RDB_BF16)
        return vs_launch<bf16_t>(dx, lddx, d->in_f, dy, lddy, d->out_f, d->sI, d->sO, coef, scale_bias, nullptr, d, num_cus, workspace, s);
    return vs_launch<float>(dx, lddx, d->in_f, dy, lddy, d->out_f, d->sI, d->sO, coef, scale_bias, nullptr, d, num_cus, workspace, s);
}

}  // namespace rdb
