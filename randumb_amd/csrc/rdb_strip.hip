// Forward of the fused linear layer, matrix-coef + bf16, "strip-stationary" algorithm:
//
//   y[t, o] = sum_i x[t, i] * W[o, i],   W = C . N,   N[m, i] = noise(PRIME*i + m, seed)
//
// A 256-thread block (one per CU) owns a strip of BO output rows and a range of tokens.
//   phase 1  builds the whole strip W[strip, 0:in] in LDS, once: every wave hashes the noise fragments of its
//            32-column blocks straight into MFMA A-operand registers and contracts them with the C rows
//            (B operand, read from L2) over k; fp32 accumulators are scaled by 2^-31, rounded to bf16 once and
//            written to LDS.  The hash (integer VALU) and the MFMAs of one block interleave in the issue stream.
//   phase 2  streams the block's tokens: each wave owns 32-row token blocks, reads x fragments directly from
//            global memory into MFMA A-operand registers (one chunk of 64 columns ahead of the math) and the W
//            fragments from LDS.  No LDS writes and no barriers in this phase.
// W never leaves the chip.  Replaces materialize() + dense product (src/rten_cpp/RandumbTensor.py:942-946, 771-791).
#include <stdlib.h>
#include "rdb_tile.hpp"

namespace rdb {

struct StripParams {
    const bf16_t *x;
    bf16_t *y;
    const void *coef;        // [out_f x k], bf16 or fp32
    const void *scale_bias;  // NULL or one value of coef dtype
    const bf16_t *bias;      // NULL or [out_f]
    int64_t ldx, ldy;
    int tokens, in_f, out_f, k;
    int in_pad;    // LDS row length in elements: in_f rounded up to 64, plus 8
    int splits;    // token ranges per strip
    int coef_dtype;
    int coef_vec;  // 16-byte loads of coef rows allowed
    uint32_t seed;
};

union Pack8 {
    bf16x8 v;
    uint32_t u[4];
};

// 8 consecutive coef values C[row, m0 .. m0+7] as bf16.
// CMODE 0: bf16 rows, 16-byte aligned, k % 16 == 0.  CMODE 1: fp32 rows, same conditions.  Both read unconditionally:
// the caller clamps `row` into the matrix (rows past out_f produce weight rows nobody reads).
// CMODE 2: any layout, element by element, zero outside the matrix.
template <int CMODE> __device__ __forceinline__ bf16x8 load_coef8(const StripParams &p, int row, int m0)
{
    Pack8 r;
    if constexpr (CMODE == 0) {
        r.v = *reinterpret_cast<const bf16x8 *>((const bf16_t *)p.coef + (int64_t)row * p.k + m0);
    } else if constexpr (CMODE == 1) {
        const float *c = (const float *)p.coef + (int64_t)row * p.k + m0;
        const f32x4 a = *reinterpret_cast<const f32x4 *>(c), b = *reinterpret_cast<const f32x4 *>(c + 4);
        r.u[0] = f32x2_to_bf16x2(a[0], a[1]);
        r.u[1] = f32x2_to_bf16x2(a[2], a[3]);
        r.u[2] = f32x2_to_bf16x2(b[0], b[1]);
        r.u[3] = f32x2_to_bf16x2(b[2], b[3]);
    } else {
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float v = load_as_f32(p.coef, p.coef_dtype, (int64_t)row * p.k + (m0 + e < p.k ? m0 + e : 0));
            f[e] = (m0 + e < p.k) ? v : 0.0f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) r.u[e] = f32x2_to_bf16x2(f[2 * e], f[2 * e + 1]);
    }
    return r.v;
}

// Noise fragment: values 2^31 * noise(i, m0 + e), e = 0..7, as bf16 (the 2^-31 is applied to the accumulator).
// `first` is the first-round hash state of (i, m0).
__device__ __forceinline__ bf16x8 noise_frag(uint32_t first)
{
    // the eight hash chains advance in lock step so that consecutive instructions are independent
    uint32_t b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = first + (uint32_t)e * SQ5_N1;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] ^= b[e] >> 9;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] += SQ5_N2;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] ^= b[e] >> 11;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] *= SQ5_N3;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] ^= b[e] >> 13;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] += SQ5_N4;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] ^= b[e] >> 15;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] *= SQ5_N5;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] ^= b[e] >> 17;
    Pack8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
    return r.v;
}

template <int BO, int MI, int CMODE>
__global__ __launch_bounds__(256, 1) void linear_fwd_strip_kernel(StripParams p)
{
    constexpr int OB = BO / 32;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *Wl = reinterpret_cast<bf16_t *>(smem_raw);  // [BO][in_pad]
    const int t = threadIdx.x, wave = t / 64, lane = t % 64, r = lane % 32, g = lane / 32;
    const int strip = blockIdx.x / p.splits, split = blockIdx.x % p.splits;
    const int o0 = strip * BO;
    const int in_pad = p.in_pad;
    const int nib = (in_pad - 8) / 32;  // 32-column blocks of the strip (in_f rounded up to 64)

    // ------------------------------------------------------------------ phase 1: W strip -> LDS
    {
        const float sb = p.scale_bias ? load_as_f32(p.scale_bias, p.coef_dtype, 0) : 0.0f;
        // coef rows of this lane, clamped into the matrix (CMODE 2 zero-fills instead)
        int crow[OB];
#pragma unroll
        for (int ob = 0; ob < OB; ++ob) {
            const int o = o0 + ob * 32 + r;
            crow[ob] = o < p.out_f ? o : p.out_f - 1;
        }
        const int ksteps = (p.k + 15) / 16;
        // CMODE 0/1: coef fragments run 4 k-steps ahead of their use in a ring of registers; the ring wraps from the last
        // k-step of one column block to the first of the next (C does not depend on the column block).
        constexpr bool RING = CMODE != 2;
        bf16x8 ring[4][OB];
        if constexpr (RING) {
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int ob = 0; ob < OB; ++ob) ring[u][ob] = load_coef8<CMODE>(p, crow[ob], (u % ksteps) * 16 + g * 8);
        }
        for (int ib = wave; ib < nib; ib += 4) {
            f32x16 acc[OB];
#pragma unroll
            for (int ob = 0; ob < OB; ++ob) acc[ob] = zero16();
            // lane (r, g) hashes column i = ib*32 + r, coefficients m = kk*16 + g*8 + e
            uint32_t first = (uint32_t)(ib * 32 + r) * PN1 + (uint32_t)(g * 8) * SQ5_N1 + p.seed;
            if constexpr (RING) {
                for (int ks = 0; ks < ksteps; ks += 4) {  // ksteps % 4 == 0 (checked on the host)
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const bf16x8 nf = noise_frag(first);
                        first += 16u * SQ5_N1;
#pragma unroll
                        for (int ob = 0; ob < OB; ++ob)
                            acc[ob] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nf, ring[u][ob], acc[ob], 0, 0, 0);
                        int nxt = ks + u + 4;
                        if (nxt >= ksteps) nxt -= ksteps;
#pragma unroll
                        for (int ob = 0; ob < OB; ++ob) ring[u][ob] = load_coef8<CMODE>(p, crow[ob], nxt * 16 + g * 8);
                    }
                }
            } else {
                for (int ks = 0; ks < ksteps; ++ks) {
                    bf16x8 cf[OB];
#pragma unroll
                    for (int ob = 0; ob < OB; ++ob) {
                        cf[ob] = load_coef8<2>(p, crow[ob], ks * 16 + g * 8);
                        if (o0 + ob * 32 + r >= p.out_f) {
                            Pack8 z;
                            z.u[0] = z.u[1] = z.u[2] = z.u[3] = 0u;
                            cf[ob] = z.v;
                        }
                    }
                    const bf16x8 nf = noise_frag(first);
                    first += 16u * SQ5_N1;
#pragma unroll
                    for (int ob = 0; ob < OB; ++ob) acc[ob] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nf, cf[ob], acc[ob], 0, 0, 0);
                }
            }
            // acc[ob][j] = 2^31 * W[o = o0 + ob*32 + r][i = ib*32 + 8*(j/4) + 4*g + j%4]
#pragma unroll
            for (int ob = 0; ob < OB; ++ob) {
                const int o = ob * 32 + r;
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    const int i = ib * 32 + 8 * jq + 4 * g;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[ob][jq * 4 + e] * 4.656612873077392578125e-10f;
                        if (p.scale_bias) v[e] += sb * noise1d((uint32_t)(crow[ob] * p.in_f + i + e), p.seed);
                    }
                    store4<bf16_t>(Wl + o * in_pad + i, v[0], v[1], v[2], v[3]);
                }
            }
        }
    }
    __syncthreads();

    // ------------------------------------------------------------------ phase 2: stream tokens
    // token blocks of 32 rows: this block's range, then this wave's share of it
    const int nrb = (p.tokens + 31) / 32;
    const int rb_lo = (int)((int64_t)nrb * split / p.splits), rb_hi = (int)((int64_t)nrb * (split + 1) / p.splits);
    const int per_wave = (rb_hi - rb_lo + 3) / 4;
    const int w_lo = rb_lo + wave * per_wave;
    const int w_hi = (w_lo + per_wave < rb_hi) ? w_lo + per_wave : rb_hi;
    const int nchunk = (in_pad - 8) / 64;
    const int nfull = p.in_f / 64;  // chunks that need no column mask

    for (int rb = w_lo; rb < w_hi; rb += MI) {
        // row pointers; rows past the end re-read the last valid row and are never stored
        const bf16_t *xrow[MI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            int row = (rb + mi) * 32 + r;
            if (rb + mi >= w_hi || row >= p.tokens) row = p.tokens - 1;
            xrow[mi] = p.x + (int64_t)row * p.ldx + g * 32;
        }
        f32x16 acc[MI][OB];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ob = 0; ob < OB; ++ob) acc[mi][ob] = zero16();

        // within a chunk of 64 columns, k-step j of lane group g covers columns g*32 + j*8 .. +7 (for x and W alike),
        // so a lane's four fragments are 64 contiguous bytes of its row
        bf16x8 xa[2][MI][4];
        auto load_x = [&](int buf, int c) {  // chunk c lies entirely inside the row
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[buf][mi][j] = *reinterpret_cast<const bf16x8 *>(xrow[mi] + c * 64 + j * 8);
        };
        auto compute = [&](int buf, int c) {
            const bf16_t *wbase = Wl + r * in_pad + c * 64 + g * 32;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bf16x8 wb[OB];
#pragma unroll
                for (int ob = 0; ob < OB; ++ob) wb[ob] = *reinterpret_cast<const bf16x8 *>(wbase + ob * 32 * in_pad + j * 8);
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int ob = 0; ob < OB; ++ob)
                        acc[mi][ob] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[buf][mi][j], wb[ob], acc[mi][ob], 0, 0, 0);
            }
        };
        // full chunks, two per trip: the loads of one chunk are in flight while the other is multiplied.  The loop body has
        // no data-dependent branch (the last prefetch re-reads a valid chunk), which keeps the load/use distance visible to
        // the compiler's wait-count insertion.
        if (nfull > 0) {
            load_x(0, 0);
            int c = 0;
            for (; c + 2 <= nfull; c += 2) {
                load_x(1, c + 1);
                __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the math it overlaps with
                compute(0, c);
                __builtin_amdgcn_sched_barrier(0);
                load_x(0, c + 2 < nfull ? c + 2 : nfull - 1);
                __builtin_amdgcn_sched_barrier(0);
                compute(1, c + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (c < nfull) compute(0, c);
        }
        if (nchunk > nfull) {
            // ragged last chunk: read a valid segment of the same row, then select zero (in_f % 8 == 0)
            const int c = nfull;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = c * 64 + g * 32 + j * 8;
                const bool ok = col < p.in_f;
                const int off = ok ? c * 64 + j * 8 : -g * 32;
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
                    Pack8 v;
                    v.v = *reinterpret_cast<const bf16x8 *>(xrow[mi] + off);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v.u[e] = ok ? v.u[e] : 0u;
                    xa[1][mi][j] = v.v;
                }
            }
            compute(1, c);
        }

        // store: acc[mi][ob][j] = y[row = (rb+mi)*32 + 8*(j/4) + 4*g + j%4][o = o0 + ob*32 + r]
#pragma unroll
        for (int ob = 0; ob < OB; ++ob) {
            const int o = o0 + ob * 32 + r;
            if (o >= p.out_f) continue;
            const float bv = p.bias ? bf16_to_f32(p.bias[o]) : 0.0f;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                if (rb + mi >= w_hi) continue;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int row = (rb + mi) * 32 + 8 * (j / 4) + 4 * g + (j % 4);
                    if (row < p.tokens) p.y[(int64_t)row * p.ldy + o] = f32_to_bf16(acc[mi][ob][j] + bv);
                }
            }
        }
    }
}

// LDS budget of gfx950 (160 KiB per workgroup).
constexpr int LDS_BYTES = 160 * 1024;

template <int BO, int CMODE> static int launch_strip_mode(const StripParams &p, int strips, hipStream_t s)
{
    const size_t smem = (size_t)BO * p.in_pad * sizeof(bf16_t);
    auto kern = linear_fwd_strip_kernel<BO, 4, CMODE>;
    if (int rl = reserve_lds(reinterpret_cast<const void *>(kern), smem, "linear_fwd_strip_kernel")) return rl;
    kern<<<strips * p.splits, 256, smem, s>>>(p);
    return check_launch("linear_fwd_strip_kernel");
}

template <int BO> static int launch_strip(const StripParams &p, int strips, hipStream_t s)
{
    // fast coef paths need aligned rows and whole groups of four 16-wide k-steps
    const bool fast = p.coef_vec && p.k % 64 == 0;
    if (fast && p.coef_dtype == RDB_BF16) return launch_strip_mode<BO, 0>(p, strips, s);
    if (fast && p.coef_dtype == RDB_F32) return launch_strip_mode<BO, 1>(p, strips, s);
    return launch_strip_mode<BO, 2>(p, strips, s);
}

// Returns RDB_E_UNSUPPORTED (without setting an error) when the shape does not fit this algorithm.
int linear_fwd_strip(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                     const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    if (d->act_dtype != RDB_BF16 || d->coef_rows == 0) return RDB_E_UNSUPPORTED;
    if (d->in_f % 8 || ldx % 8 || ((uintptr_t)x & 15) || d->tokens < 1 || d->in_f < 1) return RDB_E_UNSUPPORTED;
    if (d->tokens > (1 << 30) || d->out_f > (1 << 30) || d->out_f * d->in_f > (1ll << 31)) return RDB_E_UNSUPPORTED;
    StripParams p;
    p.x = (const bf16_t *)x;
    p.y = (bf16_t *)y;
    p.coef = coef;
    p.scale_bias = scale_bias;
    p.bias = (const bf16_t *)bias;
    p.ldx = ldx;
    p.ldy = ldy;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.in_pad = (int)(cdiv(d->in_f, 64) * 64 + 8);
    p.coef_dtype = d->coef_dtype;
    const int ces = d->coef_dtype == RDB_BF16 ? 2 : 4;
    p.coef_vec = (((uintptr_t)coef & 15) == 0) && ((d->k * ces) % 16 == 0);
    p.seed = d->seed;
    // widest strip that fits LDS; narrower strips when that leaves compute units idle
    int bo = 0;
    for (int cand : {96, 64, 32}) {
        if ((size_t)cand * p.in_pad * sizeof(bf16_t) > (size_t)LDS_BYTES) continue;
        bo = cand;
        if (cdiv(d->out_f, cand) * cdiv(d->tokens, 128) >= num_cus) break;
    }
    if (bo == 0) return RDB_E_UNSUPPORTED;
    const int strips = (int)cdiv(d->out_f, bo);
    int splits = num_cus / strips;
    const int max_splits = (int)cdiv(d->tokens, 128);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    p.splits = splits;
    if (bo == 96) return launch_strip<96>(p, strips, s);
    if (bo == 64) return launch_strip<64>(p, strips, s);
    return launch_strip<32>(p, strips, s);
}

}  // namespace rdb
