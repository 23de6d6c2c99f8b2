// Input gradient of the fused linear layer, matrix-coef + bf16, "factored" algorithm:
//
//   dx = dy . W = dy . (C . N) = (dy . C) . N
//
// With k < in*out/(in+out) the right-hand grouping needs 2*T*k*(out+in) flops instead of 2*T*out*in + 2*out*in*k and
// forms no weight tile at all.  Two kernels on the tile engine:
//   1. t[tok, m] = sum_o dy[tok, o] * C[o, m]            (dense; t is a bf16 [tokens x k] scratch in the workspace)
//   2. dx[tok, i] = sum_m t[tok, m] * noise(PRIME*i + m)  (the noise operand is hashed straight into the pipeline's
//                                                          registers, stage by stage, interleaved with the MFMAs)
// Replaces autograd's MmBackward on the re-materialised weight (materialize() + dense product,
// src/rten_cpp/RandumbTensor.py:942-946).
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

constexpr int X_BK = 64;

// ----------------------------------------------------------------------------------------------- kernel 1: t = dy . C
// tile: 128 coefficient columns (engine rows "a") x 64 tokens (engine rows "b"), contraction over out_f.  The output is
// small (tokens x k), so the token tile is kept short to have a block for every compute unit; loads run two stages ahead.
constexpr int K1_BC = 128, K1_BT = 64;

struct DyCParams {
    const bf16_t *dy;
    const bf16_t *coef;
    bf16_t *t;
    int64_t lddy;
    int tokens, out_f, k;
    int tiles_c, tiles_t;
};

__global__ __launch_bounds__(256, 2) void dx_dyc_kernel(DyCParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, coefficient tile), coefficient tile fastest: neighbours share the dy tile
    const int w = xcd_work_item(blockIdx.x, p.tiles_c * p.tiles_t);
    if (w >= p.tiles_c * p.tiles_t) return;
    const int m0 = (w % p.tiles_c) * K1_BC, tok0 = (w / p.tiles_c) * K1_BT;
    f32x16 acc[K1_BC / 64][K1_BT / 64];
#pragma unroll
    for (int mi = 0; mi < K1_BC / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < K1_BT / 64; ++ni) acc[mi][ni] = zero16();
    // "A": C[o][m], tile rows = m (contiguous in memory), contraction index = o
    GlobalOperand<K1_BC, X_BK, M_CONT> opc = {p.coef, (int64_t)p.k, m0, p.k, p.out_f, (int64_t)p.out_f * p.k};
    // "B": dy[tok][o], contraction index contiguous
    GlobalOperand<K1_BT, X_BK, K_CONT> opdy = {p.dy, p.lddy, tok0, p.tokens, p.out_f, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
    gemm_mainloop<K1_BC, K1_BT, X_BK, 2, 2>(acc, lds, opc, opdy, 0, (p.out_f + X_BK - 1) / X_BK);
    store_tile_bf16<K1_BC, K1_BT>(acc, lds, p.t, p.k, m0, p.k, tok0, p.tokens, 1.0f, nullptr);
}

// ----------------------------------------------------------------------------------------------- kernel 2: dx = t . N
// tile: 192 input features (engine rows "a", hashed operand) x 128 tokens (engine rows "b"), contraction over k
constexpr int K2_BI = 192, K2_BT = 128;

struct TNParams {
    const bf16_t *t;
    bf16_t *dx;
    int64_t lddx;
    int tokens, in_f, k;
    int tiles_i, tiles_t;
    uint32_t seed;
};

__global__ __launch_bounds__(256, 1) void dx_tn_kernel(TNParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, feature tile), feature tile fastest: neighbours share the t tile
    const int w = xcd_work_item(blockIdx.x, p.tiles_i * p.tiles_t);
    if (w >= p.tiles_i * p.tiles_t) return;
    const int i0 = (w % p.tiles_i) * K2_BI, tok0 = (w / p.tiles_i) * K2_BT;
    f32x16 acc[K2_BI / 64][K2_BT / 64];
#pragma unroll
    for (int mi = 0; mi < K2_BI / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < K2_BT / 64; ++ni) acc[mi][ni] = zero16();
    // "A": 2^31 * noise(i, m), rows = i, contraction = m; values for m >= k meet zero rows of t
    NoiseOperandRowsAreElements<K2_BI, X_BK> opn = {i0, p.seed};
    // "B": t[tok][m]
    GlobalOperand<K2_BT, X_BK, K_CONT> opt = {p.t, (int64_t)p.k, tok0, p.tokens, p.k, (int64_t)p.tokens * p.k};
    gemm_mainloop<K2_BI, K2_BT, X_BK, 1, 1>(acc, lds, opn, opt, 0, (p.k + X_BK - 1) / X_BK);
    store_tile_bf16<K2_BI, K2_BT>(acc, lds, p.dx, p.lddx, i0, p.in_f, tok0, p.tokens, 4.656612873077392578125e-10f, nullptr);
}

// ----------------------------------------------------------------------------------------------- host side
static bool dx_factored_ok(const rdb_linear_desc *d)
{
    return d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16 && d->coef_rows != 0 && d->k % 8 == 0 && d->in_f % 8 == 0 &&
           d->out_f % 8 == 0 && d->k > 0 && d->tokens > 0 && d->tokens < (1 << 30) && d->in_f < (1 << 30) && d->out_f < (1 << 30) &&
           d->k < (1 << 24) && d->tokens * d->k < (1ll << 29) && d->out_f * d->k < (1ll << 29);
}

int64_t linear_dx_factored_workspace(const rdb_linear_desc *d)
{
    if (!dx_factored_ok(d)) return 0;
    return d->tokens * d->k * (int64_t)sizeof(bf16_t);
}

// Returns RDB_E_UNSUPPORTED (without setting an error) when the request does not fit this algorithm.
int linear_dx_factored(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias,
                       const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!dx_factored_ok(d) || scale_bias) return RDB_E_UNSUPPORTED;  // the random-bias term is not low rank
    if (!workspace || workspace_bytes < linear_dx_factored_workspace(d) || ((uintptr_t)workspace & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens * lddy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    if (lddy % 8 || lddx % 8 || ((uintptr_t)dy & 15) || ((uintptr_t)coef & 15) || ((uintptr_t)dx & 15)) return RDB_E_UNSUPPORTED;
    // only worth it when the factored form is cheaper than forming the weight
    if (d->algo == RDB_ALGO_AUTO && d->k * (d->in_f + d->out_f) >= d->in_f * d->out_f) return RDB_E_UNSUPPORTED;

    DyCParams p1;
    p1.dy = (const bf16_t *)dy;
    p1.coef = (const bf16_t *)coef;
    p1.t = (bf16_t *)workspace;
    p1.lddy = lddy;
    p1.tokens = (int)d->tokens;
    p1.out_f = (int)d->out_f;
    p1.k = (int)d->k;
    p1.tiles_c = (int)cdiv(d->k, K1_BC);
    p1.tiles_t = (int)cdiv(d->tokens, K1_BT);
    int rc = launch_engine(dx_dyc_kernel, p1, p1.tiles_c * p1.tiles_t, engine_smem<K1_BC, K1_BT, X_BK, M_CONT, K_CONT>(), s, "dx_dyc_kernel");
    if (rc) return rc;

    TNParams p2;
    p2.t = (const bf16_t *)workspace;
    p2.dx = (bf16_t *)dx;
    p2.lddx = lddx;
    p2.tokens = (int)d->tokens;
    p2.in_f = (int)d->in_f;
    p2.k = (int)d->k;
    p2.seed = d->seed;
    p2.tiles_i = (int)cdiv(d->in_f, K2_BI);
    p2.tiles_t = (int)cdiv(d->tokens, K2_BT);
    return launch_engine(dx_tn_kernel, p2, p2.tiles_i * p2.tiles_t, engine_smem<K2_BI, K2_BT, X_BK, K_CONT, K_CONT>(), s, "dx_tn_kernel");
}

}  // namespace rdb
