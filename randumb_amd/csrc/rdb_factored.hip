// Forward and coefficient gradient of the fused linear layer, matrix-coef + bf16, "factored" algorithm.
//
// W = C . N has rank k, so with k < in*out/(in+out) it is cheaper never to form a weight tile:
//   forward  y  = x . W^T   = (x . N^T) . C^T      z = x . N^T is [tokens x k], the "projection" of the activations
//   dcoef    dC = dW . N^T  = dy^T . (x . N^T) = dy^T . z
// Three kernels on the tile engine:
//   z_kernel   z[tok, m]  = sum_i x[tok, i] * noise(PRIME*i + m)   noise hashed into the pipeline, interleaved with the MFMAs
//   y_kernel   y[tok, o]  = sum_m z[tok, m] * C[o, m] (+ bias[o])  dense
//   dc_kernel  dC[o, m]  += sum_tok dy[tok, o] * z[tok, m]         dense, token range split over blocks, fp32 atomics
// z is bf16; it lives in the caller's workspace, or in a buffer the caller keeps from the forward to the backward pass (it
// is all the backward pass needs of x, at k/in_f of its size).  Replaces materialize() + dense product
// (src/rten_cpp/RandumbTensor.py:942-946) and MmBackward's dW followed by materialize_bwd (RandumbTensor.py:979-990, 304-359).
#include "rdb_blocks.hpp"
#include "rdb_stationary.hpp"

namespace rdb {

constexpr float INV_2_31 = 4.656612873077392578125e-10f;
constexpr int F_BK = 64;

// ----------------------------------------------------------------------------------------------- z = x . N^T
// tile: 32 coefficients (engine rows "a", hashed) x 256 tokens (engine rows "b"), 4 waves side by side along the tokens,
// contraction over in_f; two blocks per CU.  The noise tile is hashed once per block, so the hash work of the kernel is
// (tokens / 256) * in_f * k: the token tile is as long as the accumulators allow and the coefficient tile as short.
constexpr int KZ_BM = 32, KZ_BT = 256, KZ_WM = 1;

struct ZParams {
    const bf16_t *x;
    bf16_t *z;
    int64_t ldx;
    int tokens, in_f, k;
    int tiles_m, tiles_t;
    uint32_t seed;
};

__global__ __launch_bounds__(256, 2) void factored_z_kernel(ZParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, coefficient tile), coefficient tile fastest: neighbours share the x tile
    const int w = xcd_work_item(blockIdx.x, p.tiles_m * p.tiles_t);
    if (w >= p.tiles_m * p.tiles_t) return;
    const int m0 = (w % p.tiles_m) * KZ_BM, tok0 = (w / p.tiles_m) * KZ_BT;
    constexpr int MI = KZ_BM / (32 * KZ_WM), NI = KZ_BT / (128 / KZ_WM);
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = zero16();
    // "A": 2^31 * noise(i, m), rows = m, contraction = i; values for i >= in_f meet zero columns of x
    NoiseOperandRowsAreCoefs<KZ_BM, F_BK> opn = {m0, p.seed};
    GlobalOperand<KZ_BT, F_BK, K_CONT> opx = {p.x, p.ldx, tok0, p.tokens, p.in_f, (int64_t)(p.tokens - 1) * p.ldx + p.in_f};
    gemm_mainloop<KZ_BM, KZ_BT, F_BK, 1, 1, KZ_WM>(acc, lds, opn, opx, 0, (p.in_f + F_BK - 1) / F_BK);
    store_tile_bf16<KZ_BM, KZ_BT, KZ_WM>(acc, lds, p.z, p.k, m0, p.k, tok0, p.tokens, INV_2_31, nullptr);
    RDB_STAMP(3);
}

// ----------------------------------------------------------------------------------------------- y = z . C^T
// tile: 128 output features (engine rows "a") x 128 tokens (engine rows "b"), contraction over k; two blocks per CU, so
// one block's load latency and store phase overlap the other's matrix work (k is short: a block has few stages)
constexpr int KY_BO = 128, KY_BT = 128;

struct YParams {
    const bf16_t *z;
    const bf16_t *coef;
    const bf16_t *bias;
    bf16_t *y;
    int64_t ldy;
    int tokens, out_f, k;
    int tiles_o, tiles_t;
};

__global__ __launch_bounds__(256, 2) void factored_y_kernel(YParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, output tile), output tile fastest: neighbours share the z tile, a die shares C
    const int w = xcd_work_item(blockIdx.x, p.tiles_o * p.tiles_t);
    if (w >= p.tiles_o * p.tiles_t) return;
    const int o0 = (w % p.tiles_o) * KY_BO, tok0 = (w / p.tiles_o) * KY_BT;
    f32x16 acc[KY_BO / 64][KY_BT / 64];
#pragma unroll
    for (int mi = 0; mi < KY_BO / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < KY_BT / 64; ++ni) acc[mi][ni] = zero16();
    GlobalOperand<KY_BO, F_BK, K_CONT> opc = {p.coef, (int64_t)p.k, o0, p.out_f, p.k, (int64_t)p.out_f * p.k};
    GlobalOperand<KY_BT, F_BK, K_CONT> opz = {p.z, (int64_t)p.k, tok0, p.tokens, p.k, (int64_t)p.tokens * p.k};
    gemm_mainloop<KY_BO, KY_BT, F_BK, 1, 1>(acc, lds, opc, opz, 0, (p.k + F_BK - 1) / F_BK);
    store_tile_bf16<KY_BO, KY_BT>(acc, lds, p.y, p.ldy, o0, p.out_f, tok0, p.tokens, 1.0f, p.bias);
}

// ----------------------------------------------------------------------------------------------- y = z . C^T, k <= 256
// body in rdb_stationary.hpp: the projection of a token stays in registers, the rows of C stream through LDS
template <int KG, bool BIAS> __global__ __launch_bounds__(ST_THREADS, 1) void factored_ys_kernel(StParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    stationary_block<KG, BIAS, false>(p, smem_raw, blockIdx.x);
}

// ----------------------------------------------------------------------------------------------- dC = dy^T . z
// body in rdb_blocks.hpp (dc_block)
__global__ __launch_bounds__(256, 1) void factored_dc_kernel(DcParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    dc_block(p, reinterpret_cast<bf16_t *>(smem_raw), blockIdx.x);
}

// ----------------------------------------------------------------------------------------------- host side
// What every factored kernel needs of the layer; coef_dtype is checked by the callers that read coefficients.
static bool factored_shape_ok(const rdb_linear_desc *d)
{
    return d->act_dtype == RDB_BF16 && d->coef_rows != 0 && d->k % 8 == 0 && d->in_f % 8 == 0 && d->out_f % 8 == 0 && d->k > 0 &&
           d->tokens > 0 && d->in_f > 0 && d->out_f > 0 && d->tokens * d->k < (1ll << 29) && d->out_f * d->k < (1ll << 29);
}
static bool cheaper_factored(const rdb_linear_desc *d) { return d->k * (d->in_f + d->out_f) < d->in_f * d->out_f; }
static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

int64_t linear_projection_bytes(const rdb_linear_desc *d)
{
    return factored_shape_ok(d) ? d->tokens * d->k * (int64_t)sizeof(bf16_t) : 0;
}

// The three entry points below return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
int linear_project(void *z, const void *x, int64_t ldx, const rdb_linear_desc *d, hipStream_t s)
{
    if (!factored_shape_ok(d) || d->tokens * ldx >= (1ll << 29) || ldx % 8 || !aligned16(x) || !aligned16(z)) return RDB_E_UNSUPPORTED;
    ZParams p;
    p.x = (const bf16_t *)x;
    p.z = (bf16_t *)z;
    p.ldx = ldx;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.k = (int)d->k;
    p.seed = d->seed;
    p.tiles_m = (int)cdiv(d->k, KZ_BM);
    p.tiles_t = (int)cdiv(d->tokens, KZ_BT);
    return launch_engine(factored_z_kernel, p, p.tiles_m * p.tiles_t, engine_smem<KZ_BM, KZ_BT, F_BK, K_CONT, K_CONT>(), s, "factored_z_kernel");
}

int linear_fwd_projected(void *y, int64_t ldy, const void *z, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                         hipStream_t s)
{
    if (!factored_shape_ok(d) || d->coef_dtype != RDB_BF16 || ldy % 8 || !aligned16(y) || !aligned16(z) || !aligned16(coef))
        return RDB_E_UNSUPPORTED;
    if (d->k <= ST_KMAX && ((uintptr_t)bias & 7) == 0 && d->tokens * ldy < (1ll << 29)) {  // the contraction of a token fits in registers
        StParams q;
        q.z = (const bf16_t *)z;
        q.coef = (const bf16_t *)coef;
        q.bias = (const bf16_t *)bias;
        q.y = (bf16_t *)y;
        q.ldy = ldy;
        q.k = (int)d->k;
        q.seed = 0;
        const int items = make_stationary_grid(q, d->tokens, d->out_f, num_cus);
        const int kg = (int)cdiv(d->k, 64);
        const size_t smem = stationary_smem(kg);
        if (bias) {
            switch (kg) {
            case 1: return launch_stationary(factored_ys_kernel<1, true>, q, items, smem, s, "factored_ys_kernel<1,bias>");
            case 2: return launch_stationary(factored_ys_kernel<2, true>, q, items, smem, s, "factored_ys_kernel<2,bias>");
            case 3: return launch_stationary(factored_ys_kernel<3, true>, q, items, smem, s, "factored_ys_kernel<3,bias>");
            default: return launch_stationary(factored_ys_kernel<4, true>, q, items, smem, s, "factored_ys_kernel<4,bias>");
            }
        }
        switch (kg) {
        case 1: return launch_stationary(factored_ys_kernel<1, false>, q, items, smem, s, "factored_ys_kernel<1>");
        case 2: return launch_stationary(factored_ys_kernel<2, false>, q, items, smem, s, "factored_ys_kernel<2>");
        case 3: return launch_stationary(factored_ys_kernel<3, false>, q, items, smem, s, "factored_ys_kernel<3>");
        default: return launch_stationary(factored_ys_kernel<4, false>, q, items, smem, s, "factored_ys_kernel<4>");
        }
    }
    YParams p;
    p.z = (const bf16_t *)z;
    p.coef = (const bf16_t *)coef;
    p.bias = (const bf16_t *)bias;
    p.y = (bf16_t *)y;
    p.ldy = ldy;
    p.tokens = (int)d->tokens;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.tiles_o = (int)cdiv(d->out_f, KY_BO);
    p.tiles_t = (int)cdiv(d->tokens, KY_BT);
    return launch_engine(factored_y_kernel, p, p.tiles_o * p.tiles_t, engine_smem<KY_BO, KY_BT, F_BK, K_CONT, K_CONT>(), s, "factored_y_kernel");
}

// dcoef must have been zeroed on the same stream.
int linear_dcoef_projected(float *dcoef, const void *dy, int64_t lddy, const void *z, const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    if (!factored_shape_ok(d) || d->tokens * lddy >= (1ll << 29) || lddy % 8 || !aligned16(dy) || !aligned16(z)) return RDB_E_UNSUPPORTED;
    DcParams p;
    const int items = make_dc_params(p, dcoef, dy, lddy, z, d, num_cus);
    return launch_engine(factored_dc_kernel, p, items, engine_smem<KD_BO, KD_BM, F_BK, M_CONT, M_CONT>(), s,
                         "factored_dc_kernel");
}

// y = (x . N^T) . C^T with the projection in the workspace.
int linear_fwd_factored(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                        const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (scale_bias || d->coef_dtype != RDB_BF16 || !factored_shape_ok(d)) return RDB_E_UNSUPPORTED;  // the random-bias term is not low rank
    if (!workspace || workspace_bytes < linear_projection_bytes(d)) return RDB_E_UNSUPPORTED;
    if (d->algo == RDB_ALGO_AUTO && !cheaper_factored(d)) return RDB_E_UNSUPPORTED;
    // check everything before the first launch, so that a refusal leaves nothing half done
    if (d->tokens * ldx >= (1ll << 29) || ldx % 8 || ldy % 8 || !aligned16(x) || !aligned16(coef) || !aligned16(y) || !aligned16(workspace))
        return RDB_E_UNSUPPORTED;
    int rc = linear_project(workspace, x, ldx, d, s);
    if (rc) return rc;
    return linear_fwd_projected(y, ldy, workspace, coef, bias, d, num_cus, s);
}

// dC = dy^T . (x . N^T) with the projection in the workspace; dcoef must have been zeroed on the same stream.
int linear_dcoef_factored(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus,
                          void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!factored_shape_ok(d)) return RDB_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < linear_projection_bytes(d)) return RDB_E_UNSUPPORTED;
    if (d->algo == RDB_ALGO_AUTO && !cheaper_factored(d)) return RDB_E_UNSUPPORTED;
    if (d->tokens * ldx >= (1ll << 29) || d->tokens * lddy >= (1ll << 29) || ldx % 8 || lddy % 8 || !aligned16(x) || !aligned16(dy) ||
        !aligned16(workspace))
        return RDB_E_UNSUPPORTED;
    int rc = linear_project(workspace, x, ldx, d, s);
    if (rc) return rc;
    return linear_dcoef_projected(dcoef, dy, lddy, workspace, d, num_cus, s);
}

}  // namespace rdb
