/*
 * CPU oracle for the RANDUMB pseudorandom-matrix hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may call into this
 * file: it exists so that tests, the smoke check and the CPU-baseline leg of
 * the benchmark have an independent restatement of the reference arithmetic to
 * compare the HIP kernels against.  Plain C99 (+ optional OpenMP), no GPU.
 *
 * Every function cites the reference source it restates
 * (paths relative to the reference checkout):
 *   R.py  = src/rten_cpp/RandumbTensor.py
 *   R.cu  = src/rten_cpp/csrc/cuda/rten.cu
 *
 * Pinning status (what independent evidence fixes each function):
 *   rdbo_sq5_u32 / rdbo_sq5_f32 : known-answer table + NumPy + big-int Python
 *                                 restatements + range/edge cases   -> pinned
 *   rdbo_noise_*                : reduces to rdbo_sq5_f32            -> pinned
 *   rdbo_materialize_fwd        : unit-vector coef, zero coef, linearity,
 *                                 transpose-stride identity, dense fp64
 *                                 Noise@c brute force                -> pinned
 *   rdbo_materialize_bwd        : unit-vector dW, adjoint identity,
 *                                 dense fp64 brute force             -> pinned
 *   rdbo_scale_bias_bwd         : closed form <dW, noise1d>          -> pinned
 *   rdbo_embed_fwd / _bwd       : row gather of materialize_fwd,
 *                                 adjoint identity                   -> pinned
 * The reference holds no golden vectors, tests or fixtures for this path, and
 * its CUDA/Triton sources cannot be built in a ROCm-only image, so there is no
 * oracle/_ref build.
 */
#include <stdint.h>
#include <stddef.h>
#include <math.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define SQ5_BIT_NOISE1 0xd2a80a3fu
#define SQ5_BIT_NOISE2 0xa884f197u
#define SQ5_BIT_NOISE3 0x6C736F4Bu
#define SQ5_BIT_NOISE4 0xB79F3ABBu
#define SQ5_BIT_NOISE5 0x1b56c4f5u
#define RDB_PRIME      198491317u

/* Five-round Squirrel5 bit mangle.  R.py:148-159 (2-D), R.py:216-227 (1-D),
 * R.cu:33-44.  All arithmetic is modulo 2^32. */
uint32_t rdbo_sq5_u32(uint32_t idx, uint32_t seed)
{
    uint32_t b = idx;
    b *= SQ5_BIT_NOISE1;
    b += seed;
    b ^= (b >> 9);
    b += SQ5_BIT_NOISE2;
    b ^= (b >> 11);
    b *= SQ5_BIT_NOISE3;
    b ^= (b >> 13);
    b += SQ5_BIT_NOISE4;
    b ^= (b >> 15);
    b *= SQ5_BIT_NOISE5;
    b ^= (b >> 17);
    return b;
}

/* Reinterpret as int32, convert to float (round to nearest even), scale by
 * fp32(1/0x7FFFFFFF) which is exactly 2^-31.  R.py:162-163, R.cu:19,47. */
float rdbo_sq5_f32(uint32_t idx, uint32_t seed)
{
    int32_t s = (int32_t)rdbo_sq5_u32(idx, seed);
    return (float)s * 4.656612873077392578125e-10f; /* 2^-31 */
}

/* Row/column mixing of the 2-D noise address.  R.py:148, R.cu:33. */
static inline uint32_t mix2d(uint32_t n, uint32_t m) { return RDB_PRIME * n + m; }

float rdbo_noise_at(uint32_t n, uint32_t m, uint32_t seed) { return rdbo_sq5_f32(mix2d(n, m), seed); }

/* Noise matrix (N, M) row-major: out[n*M+m] = noise(n, m).  R.py:78-105. */
void rdbo_noise_2d(float *out, int64_t N, int64_t M, uint32_t seed)
{
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m)
            out[n * M + m] = rdbo_sq5_f32(mix2d((uint32_t)n, (uint32_t)m), seed);
}

/* 1-D noise out[n] = sq5(n).  R.py:108-126, R.py:204-232. */
void rdbo_noise_1d(float *out, int64_t N, uint32_t seed)
{
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) out[n] = rdbo_sq5_f32((uint32_t)n, seed);
}

/*
 * Materialise a (P, Q) view with strides (sP, sQ) of a pseudorandom tensor.
 * R.py:235-290, 371-381; R.cu:74-110.
 *
 * coef_rows == 0 ("vector-coef", the reference form): one coef vector c[k];
 *     out[p*Q+q] = sum_m noise(a, m) * c[m],  a = q*sQ + p*sP        (R.py:264)
 * coef_rows  > 0 ("matrix-coef", row-batched form): coef is [coef_rows, k] and the
 *     storage offset a addresses a contiguous (coef_rows, row_len) base tensor:
 *     o = a / row_len, i = a % row_len, out = sum_m noise(i, m) * C[o, m].
 *     Row o alone is exactly a vector-coef tensor of shape (row_len,) with coef C[o,:].
 * scale_bias != NULL adds  scale_bias[0] * sq5_1d(a)                  (R.py:286-289)
 * acc_double: 1 = accumulate in double (closest to the real-number value),
 *             0 = serial fp32 fmaf in m order, as R.cu:101-104 does.
 */
void rdbo_materialize_fwd(float *out, const float *coef, int64_t coef_rows, int64_t k,
                          int64_t row_len, int64_t P, int64_t Q, int64_t sP, int64_t sQ,
                          uint32_t seed, const float *scale_bias, int acc_double)
{
    const int64_t Nw = P * Q;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < Nw; ++n) {
        const int64_t a = (n % Q) * sQ + (n / Q) * sP;
        const float *c = coef;
        uint32_t nrow = (uint32_t)a;
        if (coef_rows > 0) {
            c = coef + (a / row_len) * k;
            nrow = (uint32_t)(a % row_len);
        }
        const uint32_t base = RDB_PRIME * nrow;
        float r;
        if (acc_double) {
            double acc = 0.0;
            for (int64_t m = 0; m < k; ++m)
                acc += (double)rdbo_sq5_f32(base + (uint32_t)m, seed) * (double)c[m];
            if (scale_bias) acc += (double)scale_bias[0] * (double)rdbo_sq5_f32((uint32_t)a, seed);
            r = (float)acc;
        } else {
            float acc = 0.0f;
            for (int64_t m = 0; m < k; ++m)
                acc = fmaf(rdbo_sq5_f32(base + (uint32_t)m, seed), c[m], acc);
            if (scale_bias) acc += scale_bias[0] * rdbo_sq5_f32((uint32_t)a, seed);
            r = acc;
        }
        out[n] = r;
    }
}

/*
 * Gradient of the coefficients.  R.py:304-359, 383-390.
 * vector-coef (coef_rows == 0): dcoef[m] = sum_n noise(n, m) * dW[n], n = contiguous index.
 * matrix-coef: dW is (coef_rows, row_len) contiguous,
 *              dcoef[o*k+m] = sum_i noise(i, m) * dW[o*row_len+i].
 * Accumulates in double.
 */
void rdbo_materialize_bwd(float *dcoef, const float *dW, int64_t coef_rows, int64_t k,
                          int64_t row_len, int64_t Nw, uint32_t seed)
{
    if (coef_rows == 0) {
#pragma omp parallel for schedule(static)
        for (int64_t m = 0; m < k; ++m) {
            double acc = 0.0;
            for (int64_t n = 0; n < Nw; ++n)
                acc += (double)rdbo_sq5_f32(RDB_PRIME * (uint32_t)n + (uint32_t)m, seed) * (double)dW[n];
            dcoef[m] = (float)acc;
        }
    } else {
#pragma omp parallel for schedule(static)
        for (int64_t o = 0; o < coef_rows; ++o)
            for (int64_t m = 0; m < k; ++m) {
                double acc = 0.0;
                for (int64_t i = 0; i < row_len; ++i)
                    acc += (double)rdbo_sq5_f32(RDB_PRIME * (uint32_t)i + (uint32_t)m, seed) *
                           (double)dW[o * row_len + i];
                dcoef[o * k + m] = (float)acc;
            }
    }
}

/* ds = sum_n dW[n] * sq5_1d(n).  R.py:399-420. */
void rdbo_scale_bias_bwd(float *ds, const float *dW, int64_t Nw, uint32_t seed)
{
    double acc = 0.0;
#pragma omp parallel for reduction(+ : acc) schedule(static)
    for (int64_t n = 0; n < Nw; ++n) acc += (double)dW[n] * (double)rdbo_sq5_f32((uint32_t)n, seed);
    ds[0] = (float)acc;
}

/* Row gather of a vector-coef (num_rows, rowsize) tensor without materialising it.
 * out[j*rowsize+r] = sum_m noise(idx[j]*rowsize + r, m) * c[m].  R.py:998-1057. */
void rdbo_embed_fwd(float *out, const int64_t *idx, int64_t n_idx, const float *coef, int64_t k,
                    int64_t rowsize, uint32_t seed)
{
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < n_idx * rowsize; ++e) {
        const int64_t j = e / rowsize, r = e % rowsize;
        const uint32_t base = RDB_PRIME * (uint32_t)(idx[j] * rowsize + r);
        double acc = 0.0;
        for (int64_t m = 0; m < k; ++m)
            acc += (double)rdbo_sq5_f32(base + (uint32_t)m, seed) * (double)coef[m];
        out[e] = (float)acc;
    }
}

/* dcoef[m] = sum_{j,r} noise(idx[j]*rowsize + r, m) * dout[j*rowsize+r].  R.py:1059-1108. */
void rdbo_embed_bwd(float *dcoef, const int64_t *idx, int64_t n_idx, const float *dout, int64_t k,
                    int64_t rowsize, uint32_t seed)
{
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < k; ++m) {
        double acc = 0.0;
        for (int64_t e = 0; e < n_idx * rowsize; ++e) {
            const int64_t j = e / rowsize, r = e % rowsize;
            const uint32_t a = (uint32_t)(idx[j] * rowsize + r);
            acc += (double)rdbo_sq5_f32(RDB_PRIME * a + (uint32_t)m, seed) * (double)dout[e];
        }
        dcoef[m] = (float)acc;
    }
}

int rdbo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
