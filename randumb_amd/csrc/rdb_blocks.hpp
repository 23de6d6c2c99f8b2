// Block bodies shared by more than one kernel: the coefficient-gradient block (dC = dy^T . z), the reduction of its partial
// sums and the second block of the input gradient (dx = t . N) run as kernels of their own and side by side in the merged
// backward kernels.
#pragma once
#include "rdb_direct.hpp"
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

constexpr int B_BK = 64;

// unroll and prefetch depth (in stages of 64) of the dy stream in the coefficient gradient's contraction
#ifndef RDB_DC_TRIP
#define RDB_DC_TRIP 2
#endif
#ifndef RDB_DC_DSTG
#define RDB_DC_DSTG 2
#endif
#ifndef RDB_DC_RD
#define RDB_DC_RD 2
#endif
#ifndef RDB_DC_BK
#define RDB_DC_BK 64
#endif

// ----------------------------------------------------------------------------------------------- dC = dy^T . z
// tile: 128 output features (engine rows "a") x 128 coefficients (engine rows "b"), contraction over a token range
constexpr int KD_BO = 128, KD_BM = 128;

struct DcParams {
    const bf16_t *dy;
    const bf16_t *ztf;   // z transposed in fragment order, rows = coefficients
    int tsteps, kpad;    // of ztf: token k-steps per row block (tokens rounded up to 64, / 16), k rounded up to 64
    float *dcoef;
    float *partial;  // NULL: the token splits add into dcoef (zeroed beforehand) with atomics; else split s stores its sums
                     // into partial[s][out_f][k] and a reduction pass (red_block) writes dcoef (a single split: partial = dcoef)
    int64_t lddy;
    int tokens, out_f, k;
    int tiles_o, tiles_m, splits, tok_per_split;
};

// Stores (or adds) a block's 128 x 128 sums: acc[mi][ni][j] is o = o0 + wm*64 + mi*32 + 8*(j/4) + 4*g + j%4,
// m = m0 + wn*64 + ni*32 + r.  Partial sums go through LDS (`lds`: 64 x 68 floats per wave, free on entry) so that every
// lane stores 16 bytes of a row; atomic adds go straight from the registers (32 consecutive m per instruction).
__device__ __forceinline__ void dc_store(const DcParams &p, const f32x16 (&acc)[KD_BO / 64][KD_BM / 64], bf16_t *lds, int o0, int m0, int split)
{
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave >> 1, wn = wave & 1;
    float *out = p.partial ? p.partial + (int64_t)split * p.out_f * p.k : p.dcoef;
#ifdef RDB_DC_NO_STORE
    if (p.partial) return;
#endif
    if (p.partial) {
        // this wave's 64 (o) x 64 (m) quadrant, one 32-row half at a time: registers -> patch[o][m] (row stride 68 floats: the
        // column writes of 32 lanes and the row reads of 16 lanes both spread over the banks) -> 16-byte row pieces
        constexpr int LDP = 68;
        float *patch = reinterpret_cast<float *>(lds) + wave * 32 * LDP;
#pragma unroll
        for (int mi = 0; mi < KD_BO / 64; ++mi) {
#pragma unroll
            for (int ni = 0; ni < KD_BM / 64; ++ni)
#pragma unroll
                for (int j = 0; j < 16; ++j) patch[(8 * (j / 4) + 4 * g + (j % 4)) * LDP + ni * 32 + r] = acc[mi][ni][j];
            __builtin_amdgcn_wave_barrier();   // LDS serves a wave's instructions in order: the reads see these writes
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int row = q * 4 + (lane >> 4), col = (lane & 15) * 4;   // 16 lanes cover a row of 64 floats
                const int o = o0 + wm * 64 + mi * 32 + row, m = m0 + wn * 64 + col;
                const f32x4 v = *reinterpret_cast<const f32x4 *>(patch + row * LDP + col);
                if (o < p.out_f && m < p.k) *reinterpret_cast<f32x4 *>(out + (int64_t)o * p.k + m) = v;   // k is a multiple of 8
            }
            __builtin_amdgcn_wave_barrier();
        }
        return;
    }
#pragma unroll
    for (int ni = 0; ni < KD_BM / 64; ++ni) {
        const int m = m0 + wn * 64 + ni * 32 + r;
        if (m >= p.k) continue;
#pragma unroll
        for (int mi = 0; mi < KD_BO / 64; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int o = o0 + wm * 64 + mi * 32 + 8 * (j / 4) + 4 * g + (j % 4);
                if (o < p.out_f) unsafeAtomicAdd(out + (int64_t)o * p.k + m, acc[mi][ni][j]);
            }
    }
}

// `block`: index of this block among the blocks that run this body.  z comes from its transposed, fragment-ordered copy
// straight into registers: only dy passes through LDS.
__device__ __forceinline__ void dc_block_direct(const DcParams &p, bf16_t *lds, int block)
{
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, wm = wave >> 1, wn = wave & 1;
    const int total = p.tiles_o * p.tiles_m * p.splits;
    const int w = xcd_work_item(block, total);
    if (w >= total) return;
    const int m0 = (w % p.tiles_m) * KD_BM, o0 = ((w / p.tiles_m) % p.tiles_o) * KD_BO, split = w / (p.tiles_m * p.tiles_o);
    const int t_begin = split * p.tok_per_split;
    const int t_end = (t_begin + p.tok_per_split < p.tokens) ? t_begin + p.tok_per_split : p.tokens;
    f32x16 acc[KD_BO / 64][KD_BM / 64];
#pragma unroll
    for (int mi = 0; mi < KD_BO / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < KD_BM / 64; ++ni) acc[mi][ni] = zero16();
    // staged "A": dy[tok][o], tile rows = o (contiguous in memory), contraction = tokens
    GlobalOperand<KD_BO, RDB_DC_BK, M_CONT> opdy = {p.dy, p.lddy, o0, p.out_f, t_end, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
    // direct "B": z^T fragments of this wave's 64 coefficients
    FragSource fz;
    fz.init(p.ztf, (int64_t)p.kpad * p.tsteps * 16, p.tsteps, (m0 + wn * 64) >> 5, lane);
    direct_mainloop<KD_BO / 64, KD_BM / 64, RDB_DC_BK / 16, true, RDB_DC_TRIP, RDB_DC_DSTG, RDB_DC_RD>(acc, lds, opdy, fz, t_begin, (t_end - t_begin + RDB_DC_BK - 1) / RDB_DC_BK,
                                                                                                     wm * 64, lane);
    dc_store(p, acc, lds, o0, m0, split);
    RDB_STAMP(3);
}

// ----------------------------------------------------------------------------------------------- dC = sum of the splits' partial sums
// Added in split order, so the result does not depend on how the blocks were scheduled.
struct RedParams {
    const float *partial;  // [splits][n]
    float *out;            // [n]
    int64_t n;             // multiple of 4
    int splits;
    int accumulate;        // 0: out = sum of the splits; 1: out += that sum (a later chunk of tokens of the same layer)
    int out_bf16;          // 1: out is bf16, the fp32 sum rounded once (not with accumulate)
};

__device__ __forceinline__ void red_block(const RedParams &p, int block, int nblocks)
{
    const int64_t n4 = p.n / 4;
    RDB_STAMP(0);
    for (int64_t e = (int64_t)block * blockDim.x + threadIdx.x; e < n4; e += (int64_t)nblocks * blockDim.x) {
        const f32x4 *src = reinterpret_cast<const f32x4 *>(p.partial) + e;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (p.accumulate) v = reinterpret_cast<const f32x4 *>(p.out)[e];
        // eight loads in flight at a time (a loop of single loads would wait out the memory latency once per split);
        // the additions stay in split order
        for (int s0 = 0; s0 < p.splits; s0 += 8) {
            f32x4 u[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int sidx = s0 + j < p.splits ? s0 + j : p.splits - 1;   // clamped: loaded, not added
                u[j] = src[(int64_t)sidx * n4];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (s0 + j < p.splits) v += u[j];
        }
        if (p.out_bf16) {
            const uint2 h = {f32x2_to_bf16x2(v[0], v[1]), f32x2_to_bf16x2(v[2], v[3])};
            reinterpret_cast<uint2 *>(p.out)[e] = h;
        } else {
            reinterpret_cast<f32x4 *>(p.out)[e] = v;
        }
    }
    RDB_STAMP(3);
}

// ----------------------------------------------------------------------------------------------- kernel 2: dx = t . N
// tile: 64 input features (engine rows "a", hashed operand) x 256 tokens (engine rows "b"), 4 waves side by side along the
// tokens, contraction over k.  The noise tile is hashed once per block: a long token tile halves the hash work of a 128-token one.
constexpr int K2_BI = 64, K2_BT = 256, K2_WM = 1;

struct TNParams {
    const bf16_t *t;
    bf16_t *dx;
    int64_t lddx;
    int tokens, in_f, k;
    int tiles_i, tiles_t;
    uint32_t seed;
};

__device__ __forceinline__ void tn_block(const TNParams &p, bf16_t *lds, int block)
{
    // work item = (token tile, feature tile), feature tile fastest: neighbours share the t tile
    const int w = xcd_work_item(block, p.tiles_i * p.tiles_t);
    if (w >= p.tiles_i * p.tiles_t) return;
    const int i0 = (w % p.tiles_i) * K2_BI, tok0 = (w / p.tiles_i) * K2_BT;
    constexpr int MI = K2_BI / (32 * K2_WM), NI = K2_BT / (128 / K2_WM);
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = zero16();
    // "A": 2^31 * noise(i, m), rows = i, contraction = m; values for m >= k meet zero rows of t
    NoiseOperandRowsAreElements<K2_BI, B_BK> opn = {i0, p.seed};
    // "B": t[tok][m]
    GlobalOperand<K2_BT, B_BK, K_CONT> opt = {p.t, (int64_t)p.k, tok0, p.tokens, p.k, (int64_t)p.tokens * p.k};
    gemm_mainloop<K2_BI, K2_BT, B_BK, 1, 1, K2_WM>(acc, lds, opn, opt, 0, (p.k + B_BK - 1) / B_BK);
    store_tile_bf16<K2_BI, K2_BT, K2_WM>(acc, lds, p.dx, p.lddx, i0, p.in_f, tok0, p.tokens, 4.656612873077392578125e-10f, nullptr);
    RDB_STAMP(3);
}

// ----------------------------------------------------------------------------------------------- host side
// Parameters of the coefficient-gradient blocks for layer d; the token range is split so that tiles x splits is about one
// block per compute unit.  Returns the number of work items.
inline int make_dc_params(DcParams &p, float *dcoef, const void *dy, int64_t lddy, const rdb_linear_desc *d, int num_cus)
{
    p.dy = (const bf16_t *)dy;
    p.ztf = nullptr;
    p.tsteps = 0;
    p.kpad = 0;
    p.dcoef = dcoef;
    p.partial = nullptr;
    p.lddy = lddy;
    p.tokens = (int)d->tokens;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.tiles_o = (int)cdiv(d->out_f, KD_BO);
    p.tiles_m = (int)cdiv(d->k, KD_BM);
    int splits = num_cus / (p.tiles_o * p.tiles_m);
    const int max_splits = (int)cdiv(d->tokens, 256);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    p.tok_per_split = (int)(cdiv(cdiv(d->tokens, splits), B_BK) * B_BK);
    p.splits = (int)cdiv(d->tokens, p.tok_per_split);
    return p.tiles_o * p.tiles_m * p.splits;
}

// The same products on 256-wide tiles, one persistent block per compute unit (rdb_big.hip): whether they apply to a layer's
// forward product / first backward launch, and the launches.  `dc`: where the coefficient gradient's sums are stored.
bool big_fwd_applies(const rdb_linear_desc *d, int num_cus);
bool big_bwd_applies(const rdb_linear_desc *d, int num_cus);
int linear_fwd_big(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus, hipStream_t s);
int linear_bwd_big(void *t, float *dc, const void *dy, int64_t lddy, const void *state, const void *coef, const rdb_linear_desc *d, int num_cus,
                   bool want_t, bool want_dc, hipStream_t s);
void set_big_tiles_mode(int mode);
int big_tiles_mode();

inline int make_tn_params(TNParams &p, void *dx, int64_t lddx, const void *t, const rdb_linear_desc *d)
{
    p.t = (const bf16_t *)t;
    p.dx = (bf16_t *)dx;
    p.lddx = lddx;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.k = (int)d->k;
    p.seed = d->seed;
    p.tiles_i = (int)cdiv(d->in_f, K2_BI);
    p.tiles_t = (int)cdiv(d->tokens, K2_BT);
    return p.tiles_i * p.tiles_t;
}

}  // namespace rdb
