// Coefficient gradient of the fused linear layer, matrix-coef + bf16, optimised kernel:
//
//   dC[o, m] = sum_i dW[o, i] * noise(PRIME*i + m),   dW[o, i] = sum_t dy[t, o] * x[t, i]
//
// A block owns a 192 (i) x 192 (o) tile of dW and a range of tokens.  The tile is accumulated over the tokens on the
// matrix cores (both operands are read with the tile index contiguous and transposed on their way out of LDS), rounded
// once to bf16 into LDS, and immediately contracted with noise hashed on the spot - 64 coefficients at a time - again
// on the matrix cores.  Partial sums of different blocks are combined with coalesced fp32 atomics.  dW never reaches
// memory.  Replaces MmBackward's dense dW + RandumbTensorConstructor.backward -> materialize_bwd / scale_bias_bwd
// (src/rten_cpp/RandumbTensor.py:979-990, 304-359, 399-420).
#include <stdlib.h>
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

constexpr int DC_BI = 192, DC_BO = 192, DC_BK = 64, DC_MC = 64;

struct DcoefParams {
    const bf16_t *dy;
    const bf16_t *x;
    float *dcoef;
    float *dsb;
    int64_t lddy, ldx;
    int tokens, in_f, out_f, k;
    int tok_per_split, tiles_i, tiles_o, splits;
    uint32_t seed;
};

__global__ __launch_bounds__(256, 1) void linear_dcoef_fast_kernel(DcoefParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave >> 1, wn = wave & 1;
    // work item = (token split, o tile, i tile), i fastest: neighbours share the dy stream, a whole die shares the x stream
    const int w = xcd_work_item(blockIdx.x, p.tiles_i * p.tiles_o * p.splits);
    if (w >= p.tiles_i * p.tiles_o * p.splits) return;
    const int i0 = (w % p.tiles_i) * DC_BI, o0 = ((w / p.tiles_i) % p.tiles_o) * DC_BO, split = w / (p.tiles_i * p.tiles_o);
    const int t_begin = split * p.tok_per_split;
    const int t_end = (t_begin + p.tok_per_split < p.tokens) ? t_begin + p.tok_per_split : p.tokens;

    // main product: D[m = i][n = o] (x rows as the "A" tile, dy rows as the "B" tile), contraction over tokens
    f32x16 acc[DC_BI / 64][DC_BO / 64];
#pragma unroll
    for (int mi = 0; mi < DC_BI / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < DC_BO / 64; ++ni) acc[mi][ni] = zero16();
    GlobalOperand<DC_BI, DC_BK, M_CONT> opx = {p.x, p.ldx, i0, p.in_f, t_end, (int64_t)(p.tokens - 1) * p.ldx + p.in_f};
    GlobalOperand<DC_BO, DC_BK, M_CONT> opdy = {p.dy, p.lddy, o0, p.out_f, t_end, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
    gemm_mainloop<DC_BI, DC_BO, DC_BK, 1, 1>(acc, lds, opx, opdy, t_begin, (t_end - t_begin + DC_BK - 1) / DC_BK);

    // dW tile -> LDS as Ws[o][i] (bf16, i contiguous).  acc[mi][ni][j]: i = wm*96 + mi*32 + 8*(j/4) + 4*g + j%4, o = wn*96 + ni*32 + r
    constexpr int LDW = DC_BI + 8;
    bf16_t *Ws = lds;                  // [DC_BO][LDW]
    bf16_t *Ns = lds + DC_BO * LDW;    // [DC_MC][LDW]   Ns[m][i] = 2^31 * noise(i, m)
#pragma unroll
    for (int mi = 0; mi < DC_BI / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < DC_BO / 64; ++ni) {
            const int o = wn * 96 + ni * 32 + r;
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const int i = wm * 96 + mi * 32 + 8 * jq + 4 * g;
                store4<bf16_t>(Ws + o * LDW + i, acc[mi][ni][jq * 4 + 0], acc[mi][ni][jq * 4 + 1], acc[mi][ni][jq * 4 + 2],
                               acc[mi][ni][jq * 4 + 3]);
            }
        }
    __syncthreads();

    // contraction with the noise, 64 coefficients per pass: E[o][m] = sum_i Ws[o][i] * Ns[m][i]
    // wave -> coefficient block (wave & 1) and three of the six 32-row o blocks
    const int mb = wave & 1, ob0 = (wave >> 1) * 3;
    for (int mc = 0; mc < p.k; mc += DC_MC) {
        // hash: 64 x 192 values in groups of 8 consecutive i
#pragma unroll
        for (int q = 0; q < DC_MC * DC_BI / 8 / 256; ++q) {
            const int grp = q * 256 + t;
            const int mm = grp / (DC_BI / 8), i8 = (grp % (DC_BI / 8)) * 8;
            uint32_t b[8];
            const uint32_t first = (uint32_t)(i0 + i8) * PN1 + (uint32_t)(mc + mm) * SQ5_N1 + p.seed;
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * PN1);
            Frag8 f;
#pragma unroll
            for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
            *reinterpret_cast<f32x4 *>(Ns + mm * LDW + i8) = f.f4;
        }
        __syncthreads();
        f32x16 e16[3];
#pragma unroll
        for (int u = 0; u < 3; ++u) e16[u] = zero16();
#pragma unroll
        for (int ks = 0; ks < DC_BI / 16; ++ks) {
            const bf16x8 fn = *reinterpret_cast<const bf16x8 *>(Ns + (mb * 32 + r) * LDW + ks * 16 + g * 8);
#pragma unroll
            for (int u = 0; u < 3; ++u) {
                const bf16x8 fw = *reinterpret_cast<const bf16x8 *>(Ws + ((ob0 + u) * 32 + r) * LDW + ks * 16 + g * 8);
                e16[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw, fn, e16[u], 0, 0, 0);
            }
        }
        // e16[u][j]: o = (ob0+u)*32 + 8*(j/4) + 4*g + j%4, m = mc + mb*32 + r  (32 consecutive m per half wave: coalesced)
        const int m = mc + mb * 32 + r;
        if (m < p.k) {
#pragma unroll
            for (int u = 0; u < 3; ++u)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int o = o0 + (ob0 + u) * 32 + 8 * (j / 4) + 4 * g + (j % 4);
                    if (o < p.out_f) unsafeAtomicAdd(p.dcoef + (int64_t)o * p.k + m, e16[u][j] * 4.656612873077392578125e-10f);
                }
        }
        __syncthreads();
    }

    if (p.dsb) {  // d scale_bias += sum dW[o, i] * noise(o*in_f + i)
        float s = 0.0f;
        for (int e = t; e < DC_BO * DC_BI; e += 256) {
            const int oo = e / DC_BI, ii = e % DC_BI;
            s = fmaf(bf16_to_f32(Ws[oo * LDW + ii]), noise1d((uint32_t)((o0 + oo) * p.in_f + i0 + ii), p.seed), s);
        }
        float *red = reinterpret_cast<float *>(Ns);
        red[t] = s;
        __syncthreads();
        for (int st = 128; st > 0; st >>= 1) {
            if (t < st) red[t] += red[t + st];
            __syncthreads();
        }
        if (t == 0) unsafeAtomicAdd(p.dsb, red[0]);
    }
}

// Returns RDB_E_UNSUPPORTED (without setting an error) when the shape does not fit this kernel.  dcoef / dsb must have
// been zeroed by the caller on the same stream.
int linear_dcoef_fast(float *dcoef, float *dsb, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d,
                      int num_cus, hipStream_t s)
{
    if (d->act_dtype != RDB_BF16 || d->coef_rows == 0) return RDB_E_UNSUPPORTED;
    if (d->in_f % 8 || d->out_f % 8 || ldx % 8 || lddy % 8 || ((uintptr_t)x & 15) || ((uintptr_t)dy & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens < 1 || d->tokens > (1 << 30) || d->out_f > (1 << 30) || d->in_f > (1 << 30) || d->out_f * d->in_f > (1ll << 31) ||
        d->tokens * lddy >= (1ll << 29) || d->tokens * ldx >= (1ll << 29))
        return RDB_E_UNSUPPORTED;
    DcoefParams p;
    p.dy = (const bf16_t *)dy;
    p.x = (const bf16_t *)x;
    p.dcoef = dcoef;
    p.dsb = dsb;
    p.lddy = lddy;
    p.ldx = ldx;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.seed = d->seed;
    const int ti = (int)cdiv(d->in_f, DC_BI), to = (int)cdiv(d->out_f, DC_BO);
    int splits = num_cus / (ti * to);
    const int max_splits = (int)cdiv(d->tokens, 256);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    p.tok_per_split = (int)(cdiv(cdiv(d->tokens, splits), DC_BK) * DC_BK);
    splits = (int)cdiv(d->tokens, p.tok_per_split);
    p.tiles_i = ti;
    p.tiles_o = to;
    p.splits = splits;
    typedef OperandTile<DC_BI, DC_BK, M_CONT> TA;
    typedef OperandTile<DC_BO, DC_BK, M_CONT> TB;
    const size_t main_bytes = 2 * (TA::LDS_ELEMS + TB::LDS_ELEMS) * sizeof(bf16_t);
    const size_t epi_bytes = (size_t)(DC_BO + DC_MC) * (DC_BI + 8) * sizeof(bf16_t);
    const size_t smem = main_bytes > epi_bytes ? main_bytes : epi_bytes;
    if (int rl = reserve_lds(reinterpret_cast<const void *>(linear_dcoef_fast_kernel), smem, "linear_dcoef_fast_kernel")) return rl;
    linear_dcoef_fast_kernel<<<xcd_grid_size(ti * to * splits), 256, smem, s>>>(p);
    return check_launch("linear_dcoef_fast_kernel");
}

}  // namespace rdb
