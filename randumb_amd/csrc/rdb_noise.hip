// Noise probes, materialise forward/backward, random-bias gradient and embedding gather for gfx950.
// These are the HBM-facing ops of the pseudorandom tensor (the fused linear kernels live in rdb_linear.hip).
#include "rdb_common.hpp"

namespace rdb {

constexpr int NT = 256;  // threads per block for every kernel in this file

// =============================================================================================== probes
// out[n*M + m] = noise(PRIME*n + m).  Reference: RandumbTensor.py:78-105.
template <typename IM>   // type of the column index: uint32_t where M < 2^31, else int64_t
__global__ __launch_bounds__(NT) void sq5_fill_2d_kernel(float *__restrict__ out, int64_t N, int64_t M, uint32_t seed)
{
    // No division and no multiplication per element: the first round's value of the thread's first element, first(n, m) =
    // n * PN1 + m * N1 + seed (mod 2^32), then a step of (S / M, S % M) elements with a carry, S = the grid's stride
    const int64_t total = N * M, S = (int64_t)gridDim.x * NT, sn = S / M;
    const IM sm = (IM)(S - sn * M), MM = (IM)M;
    int64_t e = (int64_t)blockIdx.x * NT + threadIdx.x;
    // (the one division: in 32 bits where the operands fit, a fifth of the instructions of the 64-bit one)
    const int64_t n0 = (total < (1ll << 32)) ? (int64_t)((uint32_t)e / (uint32_t)M) : e / M;
    IM m = (IM)(e - n0 * M);
    uint32_t f = sq5_first((uint32_t)n0, (uint32_t)m, seed);
    const uint32_t step = (uint32_t)sn * PN1 + (uint32_t)sm * SQ5_N1, carry = PN1 - (uint32_t)M * SQ5_N1;
    for (; e < total; e += S) {
        out[e] = sq5_unit(sq5_tail(f));
        f += step;
        m += sm;
        if (m >= MM) {
            m -= MM;
            f += carry;
        }
    }
}

// out[n] = noise(n).  Reference: RandumbTensor.py:108-126, 204-232.
__global__ __launch_bounds__(NT) void sq5_fill_1d_kernel(float *__restrict__ out, int64_t N, uint32_t seed)
{
    for (int64_t e = (int64_t)blockIdx.x * NT + threadIdx.x; e < N; e += (int64_t)gridDim.x * NT)
        out[e] = noise1d((uint32_t)e, seed);
}

// =============================================================================================== forward
// Vector-coef materialise / embedding gather: one thread per output element, coef broadcast from LDS,
// serial fp32 FMA over m (the order the reference's CUDA kernel uses, rten.cu:101-104).
// GATHER = false: a = (n % Q)*sQ + (n / Q)*sP                       (RandumbTensor.py:264)
// GATHER = true : a = idx[n / Q]*Q + n % Q   (Q = rowsize)          (RandumbTensor.py:1029)
constexpr int COEF_CHUNK = 2048;

template <bool GATHER>
__global__ __launch_bounds__(NT) void materialize_vec_kernel(float *__restrict__ out, const void *__restrict__ coef,
                                                             int coef_dtype, int64_t k, int64_t Nw, int64_t Q,
                                                             int64_t sP, int64_t sQ, uint32_t seed,
                                                             const void *__restrict__ scale_bias,
                                                             const int64_t *__restrict__ idx)
{
    __shared__ float cs[COEF_CHUNK];
    const int64_t n = (int64_t)blockIdx.x * NT + threadIdx.x;
    const bool live = n < Nw;
    uint32_t a = 0;
    if (live) {
        const int64_t p = n / Q, q = n - p * Q;
        a = GATHER ? (uint32_t)(idx[p] * Q + q) : (uint32_t)(q * sQ + p * sP);
    }
    uint32_t first = a * PN1 + seed;  // first-round value for m = 0; +N1 per step of m
    float acc = 0.0f;
    for (int64_t m0 = 0; m0 < k; m0 += COEF_CHUNK) {
        const int cnt = (int)((k - m0) < COEF_CHUNK ? (k - m0) : COEF_CHUNK);
        __syncthreads();
        for (int j = threadIdx.x; j < cnt; j += NT) cs[j] = load_as_f32(coef, coef_dtype, m0 + j);
        __syncthreads();
        if (live) {
#pragma unroll 4
            for (int j = 0; j < cnt; ++j) {
                acc = fmaf(sq5_unit(sq5_tail(first)), cs[j], acc);
                first += SQ5_N1;
            }
        }
    }
    if (live) {
        if (scale_bias) acc += load_as_f32(scale_bias, coef_dtype, 0) * noise1d(a, seed);
        out[n] = acc;
    }
}

// Matrix-coef materialise, arbitrary view: one thread per output element (no sharing of noise between rows).
__global__ __launch_bounds__(NT) void materialize_mat_generic_kernel(float *__restrict__ out, const void *__restrict__ coef,
                                                                     int coef_dtype, int64_t k, int64_t row_len,
                                                                     int64_t Nw, int64_t Q, int64_t sP, int64_t sQ,
                                                                     uint32_t seed, const void *__restrict__ scale_bias)
{
    const int64_t n = (int64_t)blockIdx.x * NT + threadIdx.x;
    if (n >= Nw) return;
    const int64_t p = n / Q, q = n - p * Q;
    const int64_t a = q * sQ + p * sP;
    const int64_t o = a / row_len, i = a - o * row_len;
    uint32_t first = (uint32_t)i * PN1 + seed;
    float acc = 0.0f;
    for (int64_t m = 0; m < k; ++m) {
        acc = fmaf(sq5_unit(sq5_tail(first)), load_as_f32(coef, coef_dtype, o * k + m), acc);
        first += SQ5_N1;
    }
    if (scale_bias) acc += load_as_f32(scale_bias, coef_dtype, 0) * noise1d((uint32_t)a, seed);
    out[n] = acc;
}

// Matrix-coef materialise of the base tensor or its transpose: W[o, i] = sum_m C[o, m] * noise(i, m).
// A block owns a 16 (o) x 64 (i) tile and walks m in chunks of 32; the noise chunk is hashed once per block
// and shared by the 16 rows through LDS.  out[o*ooS + i*oiS].
constexpr int MT_O = 16, MT_I = 64, MT_M = 32;
__global__ __launch_bounds__(NT) void materialize_mat_tiled_kernel(float *__restrict__ out, const void *__restrict__ coef,
                                                                   int coef_dtype, int64_t rows, int64_t k, int64_t row_len,
                                                                   int64_t ooS, int64_t oiS, uint32_t seed,
                                                                   const void *__restrict__ scale_bias)
{
    __shared__ float Ns[MT_M][MT_I];
    __shared__ float Cs[MT_O][MT_M + 1];
    const int t = threadIdx.x;
    const int64_t i0 = (int64_t)blockIdx.x * MT_I, o0 = (int64_t)blockIdx.y * MT_O;
    const int il = t % MT_I, og = t / MT_I;  // thread owns column il, rows og*4 .. og*4+3
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t m0 = 0; m0 < k; m0 += MT_M) {
        __syncthreads();
        // hash the noise chunk: Ns[mm][ii] = noise(i0+ii, m0+mm); 2048 values, 8 per thread
#pragma unroll
        for (int r = 0; r < (MT_M * MT_I) / NT; ++r) {
            const int e = r * NT + t;
            const int mm = e / MT_I, ii = e % MT_I;
            Ns[mm][ii] = noise2d((uint32_t)(i0 + ii), (uint32_t)(m0 + mm), seed);
        }
        for (int e = t; e < MT_O * MT_M; e += NT) {
            const int oo = e / MT_M, mm = e % MT_M;
            const int64_t o = o0 + oo, m = m0 + mm;
            Cs[oo][mm] = (o < rows && m < k) ? load_as_f32(coef, coef_dtype, o * k + m) : 0.0f;
        }
        __syncthreads();
#pragma unroll 8
        for (int mm = 0; mm < MT_M; ++mm) {
            const float nv = Ns[mm][il];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(nv, Cs[og * 4 + j][mm], acc[j]);
        }
    }
    const int64_t i = i0 + il;
    if (i >= row_len) return;
    const float sb = scale_bias ? load_as_f32(scale_bias, coef_dtype, 0) : 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t o = o0 + og * 4 + j;
        if (o >= rows) continue;
        float v = acc[j];
        if (scale_bias) v += sb * noise1d((uint32_t)(o * row_len + i), seed);
        out[o * ooS + i * oiS] = v;
    }
}

// =============================================================================================== backward
// Vector-coef coefficient gradient / embedding gradient.
//   dcoef[m] = sum_e noise(PRIME*a(e) + m) * d[e],  a(e) = e  or  idx[e / Q]*Q + e % Q.
// grid = (ceil(k/32), splits).  A block owns 32 coefficients and the elements e = split*span .. ; its 8
// thread groups take every 8th element of a 256-element stage buffer.  Each block writes one partial row;
// reduce_rows_kernel adds the rows in a fixed order, so the result is reproducible.
// Reference: RandumbTensor.py:304-359 (split-N + relaxed atomics there), 1059-1108.
template <bool GATHER>
__global__ __launch_bounds__(NT) void coef_grad_vec_kernel(float *__restrict__ partial, const void *__restrict__ d,
                                                           int d_dtype, int64_t k, int64_t Nw, int64_t span, int64_t Q,
                                                           uint32_t seed, const int64_t *__restrict__ idx)
{
    __shared__ float ds[NT];
    __shared__ uint32_t as[NT];
    __shared__ float red[8][32];
    const int t = threadIdx.x, ml = t % 32, g = t / 32;
    const int64_t m = (int64_t)blockIdx.x * 32 + ml;
    const int64_t e_begin = (int64_t)blockIdx.y * span;
    const int64_t e_end = (e_begin + span < Nw) ? e_begin + span : Nw;
    const uint32_t mterm = (uint32_t)m * SQ5_N1 + seed;
    float acc = 0.0f;
    for (int64_t e0 = e_begin; e0 < e_end; e0 += NT) {
        __syncthreads();
        const int64_t e = e0 + t;
        float dv = 0.0f;
        uint32_t a = 0;
        if (e < e_end) {
            dv = load_as_f32(d, d_dtype, e);
            if (GATHER) {
                const int64_t j = e / Q;
                a = (uint32_t)(idx[j] * Q + (e - j * Q));
            } else {
                a = (uint32_t)e;
            }
        }
        ds[t] = dv;  // zero beyond the range, so the tail adds nothing
        as[t] = a * PN1;
        __syncthreads();
#pragma unroll 4
        for (int j = 0; j < 32; ++j) {
            const int s = j * 8 + g;
            acc = fmaf(sq5_unit(sq5_tail(as[s] + mterm)), ds[s], acc);
        }
    }
    red[g][ml] = acc;
    __syncthreads();
    if (g == 0 && m < k) {
        float s = red[0][ml];
#pragma unroll
        for (int j = 1; j < 8; ++j) s += red[j][ml];
        partial[(int64_t)blockIdx.y * k + m] = s;
    }
}

// out[c] = sum_r partial[r*cols + c], rows added in index order.
__global__ __launch_bounds__(NT) void reduce_rows_kernel(float *__restrict__ out, const float *__restrict__ partial,
                                                         int64_t rows, int64_t cols)
{
    const int64_t c = (int64_t)blockIdx.x * NT + threadIdx.x;
    if (c >= cols) return;
    float s = 0.0f;
    for (int64_t r = 0; r < rows; ++r) s += partial[r * cols + c];
    out[c] = s;
}

// Matrix-coef coefficient gradient: dC[o, m] = sum_i noise(i, m) * dW[o, i].
// A block owns a 16 (o) x 64 (m) tile and walks the whole row in chunks of 32 columns (no split: reproducible).
constexpr int GB_O = 16, GB_M = 64, GB_I = 32;
__global__ __launch_bounds__(NT) void coef_grad_mat_kernel(float *__restrict__ dcoef, const void *__restrict__ dW, int dw_dtype,
                                                           int64_t rows, int64_t k, int64_t row_len, uint32_t seed)
{
    __shared__ float Ns[GB_I][GB_M];
    __shared__ float Ds[GB_O][GB_I + 1];
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.x * GB_M, o0 = (int64_t)blockIdx.y * GB_O;
    const int ml = t % GB_M, og = t / GB_M;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t i0 = 0; i0 < row_len; i0 += GB_I) {
        __syncthreads();
#pragma unroll
        for (int r = 0; r < (GB_I * GB_M) / NT; ++r) {
            const int e = r * NT + t;
            const int ii = e / GB_M, mm = e % GB_M;
            Ns[ii][mm] = noise2d((uint32_t)(i0 + ii), (uint32_t)(m0 + mm), seed);
        }
        for (int e = t; e < GB_O * GB_I; e += NT) {
            const int oo = e / GB_I, ii = e % GB_I;
            const int64_t o = o0 + oo, i = i0 + ii;
            Ds[oo][ii] = (o < rows && i < row_len) ? load_as_f32(dW, dw_dtype, o * row_len + i) : 0.0f;
        }
        __syncthreads();
#pragma unroll 8
        for (int ii = 0; ii < GB_I; ++ii) {
            const float nv = Ns[ii][ml];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(nv, Ds[og * 4 + j][ii], acc[j]);
        }
    }
    const int64_t m = m0 + ml;
    if (m >= k) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t o = o0 + og * 4 + j;
        if (o < rows) dcoef[o * k + m] = acc[j];
    }
}

// Random-bias gradient, stage 1: partial[b] = sum over the block's span of d[e]*noise(e).
// Reference: RandumbTensor.py:399-420.
__global__ __launch_bounds__(NT) void scale_bias_grad_kernel(float *__restrict__ partial, const void *__restrict__ d, int d_dtype,
                                                             int64_t Nw, int64_t span, uint32_t seed)
{
    __shared__ float red[NT];
    const int64_t b = (int64_t)blockIdx.x * span;
    const int64_t e_end = (b + span < Nw) ? b + span : Nw;
    float acc = 0.0f;
    for (int64_t e = b + threadIdx.x; e < e_end; e += NT) acc = fmaf(load_as_f32(d, d_dtype, e), noise1d((uint32_t)e, seed), acc);
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int s = NT / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

// =============================================================================================== host side
static inline int grid_for(int64_t n, int64_t cap = 1 << 20) { return (int)(cdiv(n, NT) < cap ? cdiv(n, NT) : cap); }
static bool dtype_ok(int d) { return d == RDB_F32 || d == RDB_BF16; }

static void split_plan(int64_t Nw, int64_t k, int64_t *splits, int64_t *span)
{
    // enough blocks to fill the chip (256 CUs), but spans of at least 2048 elements and a multiple of 256
    const int64_t mblocks = cdiv(k, 32);
    int64_t want = cdiv(2048, mblocks);
    int64_t s = cdiv(Nw, 2048);
    if (s > want) s = want;
    if (s < 1) s = 1;
    int64_t sp = cdiv(cdiv(Nw, s), NT) * NT;
    if (sp < NT) sp = NT;
    *span = sp;
    *splits = cdiv(Nw, sp) > 0 ? cdiv(Nw, sp) : 1;
}

// rdb_error.hip, rdb_f32.hip
int num_compute_units();
int materialize_mat_f32(float *out, const void *coef, int coef_dtype, int64_t coef_rows, int64_t k, int64_t row_len, bool transposed, uint32_t seed,
                        const void *scale_bias, int num_cus, hipStream_t s);
int64_t coef_grad_mat_f32_workspace(int64_t coef_rows, int64_t k, int64_t row_len, int num_cus);
int coef_grad_mat_f32(float *dcoef, const void *dW, int dw_dtype, int64_t coef_rows, int64_t k, int64_t row_len, uint32_t seed, void *workspace,
                      int64_t workspace_bytes, int num_cus, hipStream_t s);

}  // namespace rdb

using namespace rdb;

extern "C" int rdb_sq5_fill_2d(float *out, int64_t N, int64_t M, uint32_t seed, void *stream)
{
    if (N < 0 || M < 0) return set_error(RDB_E_SHAPE, "rdb_sq5_fill_2d: negative size N=%lld M=%lld", (long long)N, (long long)M);
    if (N == 0 || M == 0) return RDB_OK;
    if (!out) return set_error(RDB_E_NULL, "rdb_sq5_fill_2d: out is NULL");
    if (M < (1ll << 31)) sq5_fill_2d_kernel<uint32_t><<<grid_for(N * M, 8192), NT, 0, (hipStream_t)stream>>>(out, N, M, seed);
    else sq5_fill_2d_kernel<int64_t><<<grid_for(N * M, 8192), NT, 0, (hipStream_t)stream>>>(out, N, M, seed);
    return check_launch("sq5_fill_2d_kernel");
}

extern "C" int rdb_sq5_fill_1d(float *out, int64_t N, uint32_t seed, void *stream)
{
    if (N < 0) return set_error(RDB_E_SHAPE, "rdb_sq5_fill_1d: negative size N=%lld", (long long)N);
    if (N == 0) return RDB_OK;
    if (!out) return set_error(RDB_E_NULL, "rdb_sq5_fill_1d: out is NULL");
    sq5_fill_1d_kernel<<<grid_for(N, 8192), NT, 0, (hipStream_t)stream>>>(out, N, seed);
    return check_launch("sq5_fill_1d_kernel");
}

extern "C" int rdb_materialize_fwd(float *out, const void *coef, int coef_dtype, int64_t coef_rows, int64_t k, int64_t row_len,
                                   int64_t P, int64_t Q, int64_t sP, int64_t sQ, uint32_t seed, const void *scale_bias,
                                   void *stream)
{
    if (P < 0 || Q < 0 || k < 0 || coef_rows < 0)
        return set_error(RDB_E_SHAPE, "rdb_materialize_fwd: negative size P=%lld Q=%lld k=%lld rows=%lld", (long long)P,
                         (long long)Q, (long long)k, (long long)coef_rows);
    if (!dtype_ok(coef_dtype)) return set_error(RDB_E_DTYPE, "rdb_materialize_fwd: unknown coef dtype %d", coef_dtype);
    const int64_t Nw = P * Q;
    if (Nw == 0) return RDB_OK;
    if (!out || (!coef && k > 0)) return set_error(RDB_E_NULL, "rdb_materialize_fwd: out or coef is NULL");
    if (Nw > ((int64_t)1 << 38)) return set_error(RDB_E_SHAPE, "rdb_materialize_fwd: %lld elements is too many", (long long)Nw);
    hipStream_t s = (hipStream_t)stream;
    if (coef_rows == 0) {
        materialize_vec_kernel<false><<<(unsigned)cdiv(Nw, NT), NT, 0, s>>>(out, coef, coef_dtype, k, Nw, Q, sP, sQ, seed,
                                                                            scale_bias, nullptr);
        return check_launch("materialize_vec_kernel");
    }
    if (row_len <= 0) return set_error(RDB_E_SHAPE, "rdb_materialize_fwd: matrix-coef needs row_len > 0");
    // every addressed offset must fall inside the (coef_rows, row_len) base tensor
    const int64_t max_a = (P - 1) * sP + (Q - 1) * sQ;
    if (sP < 0 || sQ < 0 || max_a >= coef_rows * row_len)
        return set_error(RDB_E_SHAPE, "rdb_materialize_fwd: view (%lld,%lld)/(%lld,%lld) leaves the (%lld,%lld) base tensor",
                         (long long)P, (long long)Q, (long long)sP, (long long)sQ, (long long)coef_rows, (long long)row_len);
    const bool base = (P == coef_rows && Q == row_len && sP == row_len && sQ == 1);
    const bool transposed = (P == row_len && Q == coef_rows && sP == 1 && sQ == row_len);
    if (base || transposed) {
        // from some tens of millions of multiply-adds on: C . N on the fp32 matrix cores, the noise hashed as an operand
        const int rc = materialize_mat_f32(out, coef, coef_dtype, coef_rows, k, row_len, transposed, seed, scale_bias, num_compute_units(), s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        dim3 grid((unsigned)cdiv(row_len, MT_I), (unsigned)cdiv(coef_rows, MT_O));
        materialize_mat_tiled_kernel<<<grid, NT, 0, s>>>(out, coef, coef_dtype, coef_rows, k, row_len, base ? row_len : 1,
                                                         base ? 1 : coef_rows, seed, scale_bias);
        return check_launch("materialize_mat_tiled_kernel");
    }
    materialize_mat_generic_kernel<<<(unsigned)cdiv(Nw, NT), NT, 0, s>>>(out, coef, coef_dtype, k, row_len, Nw, Q, sP, sQ, seed,
                                                                         scale_bias);
    return check_launch("materialize_mat_generic_kernel");
}

extern "C" int64_t rdb_materialize_bwd_workspace_bytes(int64_t coef_rows, int64_t k, int64_t row_len, int64_t Nw)
{
    if (coef_rows != 0) return coef_grad_mat_f32_workspace(coef_rows, k, row_len, num_compute_units());   // matrix-coef: the ranges' sums
    if (k <= 0 || Nw <= 0) return 0;
    int64_t splits, span;
    split_plan(Nw, k, &splits, &span);
    return splits > 1 ? splits * k * (int64_t)sizeof(float) : 0;
}

static int coef_grad_vec(float *dcoef, const void *d, int d_dtype, int64_t k, int64_t Nw, int64_t Q, uint32_t seed,
                         const int64_t *idx, void *workspace, int64_t workspace_bytes, hipStream_t s, const char *who)
{
    int64_t splits, span;
    split_plan(Nw, k, &splits, &span);
    float *partial = dcoef;
    if (splits > 1) {
        if (!workspace || workspace_bytes < splits * k * (int64_t)sizeof(float))
            return set_error(RDB_E_WORKSPACE, "%s: workspace of %lld bytes needed, %lld given", who,
                             (long long)(splits * k * sizeof(float)), (long long)workspace_bytes);
        partial = (float *)workspace;
    }
    dim3 grid((unsigned)cdiv(k, 32), (unsigned)splits);
    if (idx)
        coef_grad_vec_kernel<true><<<grid, NT, 0, s>>>(partial, d, d_dtype, k, Nw, span, Q, seed, idx);
    else
        coef_grad_vec_kernel<false><<<grid, NT, 0, s>>>(partial, d, d_dtype, k, Nw, span, Q, seed, nullptr);
    int rc = check_launch("coef_grad_vec_kernel");
    if (rc || splits == 1) return rc;
    reduce_rows_kernel<<<(unsigned)cdiv(k, NT), NT, 0, s>>>(dcoef, partial, splits, k);
    return check_launch("reduce_rows_kernel");
}

extern "C" int rdb_materialize_bwd(float *dcoef, const void *dW, int dw_dtype, int64_t coef_rows, int64_t k, int64_t row_len,
                                   int64_t Nw, uint32_t seed, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (k < 0 || Nw < 0 || coef_rows < 0)
        return set_error(RDB_E_SHAPE, "rdb_materialize_bwd: negative size k=%lld Nw=%lld rows=%lld", (long long)k, (long long)Nw,
                         (long long)coef_rows);
    if (!dtype_ok(dw_dtype)) return set_error(RDB_E_DTYPE, "rdb_materialize_bwd: unknown dW dtype %d", dw_dtype);
    if (k == 0) return RDB_OK;
    if (!dcoef) return set_error(RDB_E_NULL, "rdb_materialize_bwd: dcoef is NULL");
    hipStream_t s = (hipStream_t)stream;
    if (coef_rows == 0) {
        if (Nw == 0) {  // empty sum
            reduce_rows_kernel<<<(unsigned)cdiv(k, NT), NT, 0, s>>>(dcoef, dcoef, 0, k);
            return check_launch("reduce_rows_kernel");
        }
        if (!dW) return set_error(RDB_E_NULL, "rdb_materialize_bwd: dW is NULL");
        return coef_grad_vec(dcoef, dW, dw_dtype, k, Nw, 1, seed, nullptr, workspace, workspace_bytes, s, "rdb_materialize_bwd");
    }
    if (row_len < 0 || coef_rows * row_len != Nw)
        return set_error(RDB_E_SHAPE, "rdb_materialize_bwd: Nw=%lld is not rows*row_len=%lld*%lld", (long long)Nw,
                         (long long)coef_rows, (long long)row_len);
    if (!dW && Nw > 0) return set_error(RDB_E_NULL, "rdb_materialize_bwd: dW is NULL");
    {   // large enough: dW . N^T on the fp32 matrix cores
        const int rc = coef_grad_mat_f32(dcoef, dW, dw_dtype, coef_rows, k, row_len, seed, workspace, workspace_bytes, num_compute_units(), s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    dim3 grid((unsigned)cdiv(k, GB_M), (unsigned)cdiv(coef_rows, GB_O));
    coef_grad_mat_kernel<<<grid, NT, 0, s>>>(dcoef, dW, dw_dtype, coef_rows, k, row_len, seed);
    return check_launch("coef_grad_mat_kernel");
}

static void sb_plan(int64_t Nw, int64_t *blocks, int64_t *span)
{
    int64_t b = cdiv(Nw, 4096);
    if (b > 1024) b = 1024;
    if (b < 1) b = 1;
    *span = cdiv(cdiv(Nw, b), NT) * NT;
    if (*span < NT) *span = NT;
    *blocks = cdiv(Nw, *span) > 0 ? cdiv(Nw, *span) : 1;
}

extern "C" int64_t rdb_scale_bias_bwd_workspace_bytes(int64_t Nw)
{
    if (Nw <= 0) return 0;
    int64_t blocks, span;
    sb_plan(Nw, &blocks, &span);
    return blocks > 1 ? blocks * (int64_t)sizeof(float) : 0;
}

extern "C" int rdb_scale_bias_bwd(float *ds, const void *dW, int dw_dtype, int64_t Nw, uint32_t seed, void *workspace,
                                  int64_t workspace_bytes, void *stream)
{
    if (Nw < 0) return set_error(RDB_E_SHAPE, "rdb_scale_bias_bwd: negative size %lld", (long long)Nw);
    if (!dtype_ok(dw_dtype)) return set_error(RDB_E_DTYPE, "rdb_scale_bias_bwd: unknown dW dtype %d", dw_dtype);
    if (!ds) return set_error(RDB_E_NULL, "rdb_scale_bias_bwd: ds is NULL");
    hipStream_t s = (hipStream_t)stream;
    if (Nw == 0) {
        reduce_rows_kernel<<<1, NT, 0, s>>>(ds, ds, 0, 1);
        return check_launch("reduce_rows_kernel");
    }
    if (!dW) return set_error(RDB_E_NULL, "rdb_scale_bias_bwd: dW is NULL");
    int64_t blocks, span;
    sb_plan(Nw, &blocks, &span);
    float *partial = ds;
    if (blocks > 1) {
        if (!workspace || workspace_bytes < blocks * (int64_t)sizeof(float))
            return set_error(RDB_E_WORKSPACE, "rdb_scale_bias_bwd: workspace of %lld bytes needed, %lld given",
                             (long long)(blocks * sizeof(float)), (long long)workspace_bytes);
        partial = (float *)workspace;
    }
    scale_bias_grad_kernel<<<(unsigned)blocks, NT, 0, s>>>(partial, dW, dw_dtype, Nw, span, seed);
    int rc = check_launch("scale_bias_grad_kernel");
    if (rc || blocks == 1) return rc;
    reduce_rows_kernel<<<1, NT, 0, s>>>(ds, partial, blocks, 1);
    return check_launch("reduce_rows_kernel");
}

extern "C" int rdb_embed_fwd(float *out, const int64_t *idx, int64_t n_idx, const void *coef, int coef_dtype, int64_t k,
                             int64_t rowsize, uint32_t seed, void *stream)
{
    if (n_idx < 0 || rowsize < 0 || k < 0)
        return set_error(RDB_E_SHAPE, "rdb_embed_fwd: negative size n_idx=%lld rowsize=%lld k=%lld", (long long)n_idx,
                         (long long)rowsize, (long long)k);
    if (!dtype_ok(coef_dtype)) return set_error(RDB_E_DTYPE, "rdb_embed_fwd: unknown coef dtype %d", coef_dtype);
    const int64_t Nw = n_idx * rowsize;
    if (Nw == 0) return RDB_OK;
    if (!out || !idx || (!coef && k > 0)) return set_error(RDB_E_NULL, "rdb_embed_fwd: out, idx or coef is NULL");
    materialize_vec_kernel<true><<<(unsigned)cdiv(Nw, NT), NT, 0, (hipStream_t)stream>>>(out, coef, coef_dtype, k, Nw, rowsize, 0,
                                                                                         0, seed, nullptr, idx);
    return check_launch("materialize_vec_kernel<gather>");
}

extern "C" int64_t rdb_embed_bwd_workspace_bytes(int64_t n_idx, int64_t rowsize, int64_t k)
{
    return rdb_materialize_bwd_workspace_bytes(0, k, 0, n_idx * rowsize);
}

extern "C" int rdb_embed_bwd(float *dcoef, const int64_t *idx, int64_t n_idx, const void *dout, int dout_dtype, int64_t k,
                             int64_t rowsize, uint32_t seed, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (n_idx < 0 || rowsize < 0 || k < 0)
        return set_error(RDB_E_SHAPE, "rdb_embed_bwd: negative size n_idx=%lld rowsize=%lld k=%lld", (long long)n_idx,
                         (long long)rowsize, (long long)k);
    if (!dtype_ok(dout_dtype)) return set_error(RDB_E_DTYPE, "rdb_embed_bwd: unknown dout dtype %d", dout_dtype);
    if (k == 0) return RDB_OK;
    if (!dcoef) return set_error(RDB_E_NULL, "rdb_embed_bwd: dcoef is NULL");
    hipStream_t s = (hipStream_t)stream;
    const int64_t Nw = n_idx * rowsize;
    if (Nw == 0) {
        reduce_rows_kernel<<<(unsigned)cdiv(k, NT), NT, 0, s>>>(dcoef, dcoef, 0, k);
        return check_launch("reduce_rows_kernel");
    }
    if (!idx || !dout) return set_error(RDB_E_NULL, "rdb_embed_bwd: idx or dout is NULL");
    return coef_grad_vec(dcoef, dout, dout_dtype, k, Nw, rowsize, seed, idx, workspace, workspace_bytes, s, "rdb_embed_bwd");
}
