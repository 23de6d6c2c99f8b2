// Building blocks of the general fused-linear kernels: MFMA fragments over LDS tiles, global->LDS tile
// loaders, and the on-chip generator of pseudorandom weight tiles.  gfx950 only, 256-thread blocks.
#pragma once

#include "rdb_common.hpp"

namespace rdb {

constexpr int TILE_THREADS = 256;

// ----------------------------------------------------------------------------------------------- fragments
// One "k-step" contracts 16 values of k with a 32x32 output block.  In every operand tile the contraction
// index is the contiguous one, and lane (r = lane % 32, g = lane / 32) holds k = 8g .. 8g+7 of row r, for
// the A and the B operand alike.  bf16: one v_mfma_f32_32x32x16_bf16.  fp32: eight v_mfma_f32_32x32x2_f32,
// the e-th one contracting k = e and k = 8 + e (any pairing is valid as long as A and B agree).
// Output block: acc[j] is row 8*(j/4) + 4*g + j%4, column r.
template <typename T> struct MMA;

template <> struct MMA<bf16_t> {
    typedef bf16x8 Frag;
    static constexpr int PAD = 8;  // elements; keeps 16-byte LDS reads of 32 consecutive rows conflict-free
    __device__ static __forceinline__ Frag load(const bf16_t *p) { return *reinterpret_cast<const bf16x8 *>(p); }
    __device__ static __forceinline__ void mma(f32x16 &c, const Frag &a, const Frag &b)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

template <> struct MMA<float> {
    struct Frag {
        f32x4 lo, hi;
    };
    static constexpr int PAD = 4;
    __device__ static __forceinline__ Frag load(const float *p)
    {
        Frag f;
        f.lo = *reinterpret_cast<const f32x4 *>(p);
        f.hi = *reinterpret_cast<const f32x4 *>(p + 4);
        return f;
    }
    __device__ static __forceinline__ void mma(f32x16 &c, const Frag &a, const Frag &b)
    {
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.lo[e], b.lo[e], c, 0, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.hi[e], b.hi[e], c, 0, 0, 0);
    }
};

__device__ __forceinline__ f32x16 zero16()
{
    f32x16 z;
#pragma unroll
    for (int j = 0; j < 16; ++j) z[j] = 0.0f;
    return z;
}

// ----------------------------------------------------------------------------------------------- loaders
// dst[r][c] (row stride ld) = src[(row0 + r)*ld_src + col0 + c] for r < R, c < C; zero outside
// (rows >= nrows, cols >= ncols).  C is the contraction width of the tile; src rows are contiguous in c.
template <typename T, int R, int C>
__device__ __forceinline__ void load_tile_rowmajor(T *__restrict__ dst, int ld, const T *__restrict__ src, int64_t ld_src,
                                                   int64_t row0, int64_t nrows, int64_t col0, int64_t ncols, bool vec_ok)
{
    constexpr int V = 16 / (int)sizeof(T);  // elements per 16-byte segment
    constexpr int SEGS = R * C / V;
    static_assert(SEGS % TILE_THREADS == 0 || SEGS < TILE_THREADS, "tile/thread mismatch");
    for (int s = threadIdx.x; s < SEGS; s += TILE_THREADS) {
        const int r = s / (C / V), c = (s % (C / V)) * V;
        const int64_t gr = row0 + r, gc = col0 + c;
        T *d = dst + r * ld + c;
        if (vec_ok && gr < nrows && gc + V <= ncols) {
            *reinterpret_cast<f32x4 *>(d) = *reinterpret_cast<const f32x4 *>(src + gr * ld_src + gc);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) d[e] = (gr < nrows && gc + e < ncols) ? src[gr * ld_src + gc + e] : (T)0;
        }
    }
}

// dst[r][c] = src[(k0 + c)*ld_src + row0 + r]: the tile's rows run along the contiguous axis of src, its
// contraction index c along src's rows (used when the contraction is over tokens).  Zero outside.
template <typename T, int R, int C>
__device__ __forceinline__ void load_tile_transposed(T *__restrict__ dst, int ld, const T *__restrict__ src, int64_t ld_src,
                                                     int64_t row0, int64_t nrows, int64_t k0, int64_t nk, bool vec_ok)
{
    constexpr int V = 16 / (int)sizeof(T);
    constexpr int SEGS = R * C / V;
    for (int s = threadIdx.x; s < SEGS; s += TILE_THREADS) {
        const int c = s / (R / V), r = (s % (R / V)) * V;
        const int64_t gk = k0 + c, gr = row0 + r;
        T v[V];
        if (vec_ok && gk < nk && gr + V <= nrows) {
            *reinterpret_cast<f32x4 *>(v) = *reinterpret_cast<const f32x4 *>(src + gk * ld_src + gr);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = (gk < nk && gr + e < nrows) ? src[gk * ld_src + gr + e] : (T)0;
        }
#pragma unroll
        for (int e = 0; e < V; ++e) dst[(r + e) * ld + c] = v[e];
    }
}

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

// Writes 4 consecutive elements dst[0..3] from fp32 values.
template <typename T> __device__ __forceinline__ void store4(T *dst, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4<float>(float *dst, float a, float b, float c, float d)
{
    f32x4 v = {a, b, c, d};
    *reinterpret_cast<f32x4 *>(dst) = v;
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t *dst, float a, float b, float c, float d)
{
    uint2 v;
    v.x = f32x2_to_bf16x2(a, b);
    v.y = f32x2_to_bf16x2(c, d);
    *reinterpret_cast<uint2 *>(dst) = v;
}

// ----------------------------------------------------------------------------------------------- weight tiles
// What a kernel needs to regenerate weight elements.
struct WeightSpec {
    const void *coef;        // [k] or [out_f x k]
    const void *scale_bias;  // NULL or one value (coef dtype)
    int64_t out_f, in_f, k;
    int64_t sO, sI;          // storage strides of element (o, i)
    uint32_t seed;
    int coef_dtype;
};

// Generates the RO x RI weight block at (o0, i0) into an LDS tile, as element type T (fp32 accumulation,
// one rounding to T):
//   OI = true : dst[o - o0][i - i0]   (row stride ld, i contiguous)
//   OI = false: dst[i - i0][o - o0]   (row stride ld, o contiguous)
// MATRIX = true : W[o, i] = sum_m C[o, m] * noise(i, m).  The noise chunk is hashed once per block into LDS
//                 and contracted with the coef chunk on the matrix cores.
// MATRIX = false: W[o, i] = sum_m c[m] * noise(o*sO + i*sI, m), fp32 FMA on the vector ALU.
// scratch: at least gen_scratch_elems<T, RO, RI>() elements of T.  All 256 threads must call; the tile is
// complete after the next __syncthreads().  Elements with o >= out_f are written as exact zeros when
// MATRIX (zero coef rows); other out-of-range elements hold finite values that callers cancel by zero-filling
// the operand they meet.
constexpr int GEN_KC = 32;  // coef chunk per step of the matrix-coef generator

template <typename T, int RO, int RI> __host__ __device__ constexpr int gen_scratch_elems()
{
    return (RO + RI) * (GEN_KC + MMA<T>::PAD);
}

template <typename T, int RO, int RI, bool OI, bool MATRIX>
__device__ __forceinline__ void gen_w_tile(T *__restrict__ dst, int ld, T *__restrict__ scratch, const WeightSpec &w, int64_t o0,
                                           int64_t i0)
{
    const int t = threadIdx.x;
    const float sb = w.scale_bias ? load_as_f32(w.scale_bias, w.coef_dtype, 0) : 0.0f;
    if constexpr (MATRIX) {
        constexpr int LDS = GEN_KC + MMA<T>::PAD;
        T *Cs = scratch;             // [RO][LDS]  Cs[o][m]
        T *Ns = scratch + RO * LDS;  // [RI][LDS]  Ns[i][m]
        // D[a][b] = sum_m Pa[a][m] * Pb[b][m]; a lane ends up with 4 consecutive a for one b, so b indexes the
        // rows of dst and a its contiguous axis.
        constexpr int RA = OI ? RI : RO, RB = OI ? RO : RI;
        T *Pa = OI ? Ns : Cs;
        T *Pb = OI ? Cs : Ns;
        constexpr int NBLK = (RA / 32) * (RB / 32);
        static_assert(NBLK % 4 == 0, "weight block must split into a multiple of 4 32x32 blocks");
        constexpr int PER_WAVE = NBLK / 4;
        const int wave = t / 64, lane = t % 64, r = lane % 32, g = lane / 32;
        f32x16 acc[PER_WAVE];
#pragma unroll
        for (int b = 0; b < PER_WAVE; ++b) acc[b] = zero16();
        for (int64_t m0 = 0; m0 < w.k; m0 += GEN_KC) {
            __syncthreads();  // previous chunk's fragments consumed (and dst's previous readers done)
            for (int e = t; e < RO * GEN_KC; e += TILE_THREADS) {
                const int oo = e / GEN_KC, mm = e % GEN_KC;
                const int64_t o = o0 + oo, m = m0 + mm;
                const float v = (o < w.out_f && m < w.k) ? load_as_f32(w.coef, w.coef_dtype, o * w.k + m) : 0.0f;
                Cs[oo * LDS + mm] = from_f32<T>(v);
            }
            for (int e = t; e < RI * GEN_KC; e += TILE_THREADS) {
                const int ii = e / GEN_KC, mm = e % GEN_KC;
                Ns[ii * LDS + mm] = from_f32<T>(noise2d((uint32_t)(i0 + ii), (uint32_t)(m0 + mm), w.seed));
            }
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < GEN_KC / 16; ++ks) {
#pragma unroll
                for (int b = 0; b < PER_WAVE; ++b) {
                    const int blk = wave * PER_WAVE + b;
                    const int ab = blk % (RA / 32), bb = blk / (RA / 32);
                    typename MMA<T>::Frag fa = MMA<T>::load(Pa + (ab * 32 + r) * LDS + ks * 16 + g * 8);
                    typename MMA<T>::Frag fb = MMA<T>::load(Pb + (bb * 32 + r) * LDS + ks * 16 + g * 8);
                    MMA<T>::mma(acc[b], fa, fb);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < PER_WAVE; ++b) {
            const int blk = wave * PER_WAVE + b;
            const int ab = blk % (RA / 32), bb = blk / (RA / 32);
            const int bidx = bb * 32 + r;  // row of dst
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const int a0 = ab * 32 + 8 * jq + 4 * g;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[b][jq * 4 + e];
                    if (w.scale_bias) {
                        const int64_t o = o0 + (OI ? bidx : a0 + e), i = i0 + (OI ? a0 + e : bidx);
                        if (o < w.out_f) v[e] += sb * noise1d((uint32_t)(o * w.sO + i * w.sI), w.seed);
                    }
                }
                store4<T>(dst + bidx * ld + a0, v[0], v[1], v[2], v[3]);
            }
        }
    } else {
        // vector-coef: each thread owns RO*RI/256 elements and walks m once, reading c[m] (uniform address).
        constexpr int PER = RO * RI / TILE_THREADS;
        constexpr int RC = OI ? RI : RO;  // contiguous extent of dst
        uint32_t first[PER];
        float acc[PER];
        uint32_t addr[PER];
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int lin = e * TILE_THREADS + t;
            const int rr = lin / RC, cc = lin % RC;
            const int64_t o = o0 + (OI ? rr : cc), i = i0 + (OI ? cc : rr);
            addr[e] = (uint32_t)(o * w.sO + i * w.sI);
            first[e] = addr[e] * PN1 + w.seed;
            acc[e] = 0.0f;
        }
        for (int64_t m = 0; m < w.k; ++m) {
            const float c = load_as_f32(w.coef, w.coef_dtype, m);
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                acc[e] = fmaf(sq5_unit(sq5_tail(first[e])), c, acc[e]);
                first[e] += SQ5_N1;
            }
        }
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int lin = e * TILE_THREADS + t;
            const int rr = lin / RC, cc = lin % RC;
            float v = acc[e];
            if (w.scale_bias) v += sb * noise1d(addr[e], w.seed);
            dst[rr * ld + cc] = from_f32<T>(v);
        }
    }
}

}  // namespace rdb
