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
#include "rdb_blocks.hpp"
#include "rdb_stationary.hpp"

namespace rdb {

constexpr int X_BK = 64;

// ----------------------------------------------------------------------------------------------- kernel 1: t = dy . C
// tile: 128 coefficient columns (engine rows "a") x 64 tokens (engine rows "b"), contraction over out_f.  The output is
// small (tokens x k), so the token tile is kept short to have a block for every compute unit; loads run two stages ahead.
constexpr int K1_BC = 128, K1_BT = 64;
// pipeline shape of the dy.C blocks that take C^T straight into registers: contraction per stage, stages per unrolled trip,
// how many stages ahead dy is loaded, depth of the fragment ring in stages, wave priority
#ifndef RDB_DYC_BKD
#define RDB_DYC_BKD 128
#endif
#ifndef RDB_DYC_TRIP
#define RDB_DYC_TRIP 2
#endif
#ifndef RDB_DYC_DSTG
#define RDB_DYC_DSTG 2
#endif
#ifndef RDB_DYC_RD
#define RDB_DYC_RD 1
#endif
#ifndef RDB_DYC_PRIO
#define RDB_DYC_PRIO 2
#endif

struct DyCParams {
    const bf16_t *dy;
    const bf16_t *coef;
    const bf16_t *ctf;      // NULL, or C transposed in fragment order (rows = coefficients), valid when *ctf_flag != 0
    const uint32_t *ctf_flag;
    int osteps, kpad;       // of ctf: k-steps per row block (out_f rounded up to 64, / 16), k rounded up to 64
    bf16_t *t;
    float *zero;     // NULL, or an array this launch clears on the side (16-byte aligned, zero_n a multiple of 4)
    int64_t zero_n;
    int64_t lddy;
    int tokens, out_f, k;
    int tiles_c, tiles_t;
    int frag_ksteps;  // 0: t row-major [tokens x k]; else t in fragment order with this many k-steps per 32 tokens and scaled
                      // by 2^-31, for the kernel that keeps it in registers (rdb_stationary.hpp)
};

// `block`: index of this block among the blocks that run this body.
__device__ __forceinline__ void dyc_block(const DyCParams &p, bf16_t *lds, int block)
{
    // work item = (token tile, coefficient tile), coefficient tile fastest: neighbours share the dy tile
    const int w = xcd_work_item(block, p.tiles_c * p.tiles_t);
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
    if (p.frag_ksteps)
        store_tile_bf16_frag<K1_BC, K1_BT>(acc, lds, p.t, p.frag_ksteps, m0, p.frag_ksteps * 16, tok0, (p.tokens + 31) / 32 * 32,
                                           4.656612873077392578125e-10f);
    else
        store_tile_bf16<K1_BC, K1_BT>(acc, lds, p.t, p.k, m0, p.k, tok0, p.tokens, 1.0f, nullptr);
    RDB_STAMP(3);
}

// The same block with C taken from its transposed, fragment-ordered copy: only dy passes through LDS.  The four waves split
// the coefficient rows (one 32-row block each, no fragment loaded twice) and share the 64 tokens.
__device__ __forceinline__ void dyc_block_direct(const DyCParams &p, bf16_t *lds, int block)
{
    const int w = xcd_work_item(block, p.tiles_c * p.tiles_t);
    if (w >= p.tiles_c * p.tiles_t) return;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const int m0 = (w % p.tiles_c) * K1_BC, tok0 = (w / p.tiles_c) * K1_BT;
    f32x16 acc[1][K1_BT / 32];
#pragma unroll
    for (int ni = 0; ni < K1_BT / 32; ++ni) acc[0][ni] = zero16();
    // stages of 128: half as many barriers (and waits for the first fragments after them) as with 64, for the same LDS
    constexpr int BKD = RDB_DYC_BKD;
    GlobalOperand<K1_BT, BKD, K_CONT> opdy = {p.dy, p.lddy, tok0, p.tokens, p.out_f, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
    FragSource fc;
    fc.init(p.ctf, (int64_t)p.kpad * p.osteps * 16, p.osteps, (m0 >> 5) + wave, lane);
    // these blocks are the longer ones of the launch they share with the coefficient-gradient blocks: their waves issue first
    __builtin_amdgcn_s_setprio(RDB_DYC_PRIO);
    direct_mainloop<K1_BT / 32, 1, BKD / 16, false, RDB_DYC_TRIP, RDB_DYC_DSTG, RDB_DYC_RD>(acc, lds, opdy, fc, 0, (p.out_f + BKD - 1) / BKD, 0, lane);
    if (p.frag_ksteps)
        store_tile_bf16_frag<K1_BC, K1_BT, 4>(acc, lds, p.t, p.frag_ksteps, m0, p.frag_ksteps * 16, tok0, (p.tokens + 31) / 32 * 32,
                                              4.656612873077392578125e-10f);
    else
        store_tile_bf16<K1_BC, K1_BT, 4>(acc, lds, p.t, p.k, m0, p.k, tok0, p.tokens, 1.0f, nullptr);
    RDB_STAMP(3);
}

__global__ __launch_bounds__(256, 2) void dx_dyc_kernel(DyCParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if (p.zero) {  // a kernel later in the stream accumulates into this array with atomics
        const f32x4 z4 = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < p.zero_n / 4; e += (int64_t)gridDim.x * 256)
            reinterpret_cast<f32x4 *>(p.zero)[e] = z4;
    }
    dyc_block(p, reinterpret_cast<bf16_t *>(smem_raw), blockIdx.x);
}

// ----------------------------------------------------------------------------------------------- kernel 2: dx = t . N
// body in rdb_blocks.hpp (tn_block)
__global__ __launch_bounds__(256, 1) void dx_tn_kernel(TNParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    tn_block(p, reinterpret_cast<bf16_t *>(smem_raw), blockIdx.x);
}

// ----------------------------------------------------------------------------------------------- dC and dx = t . N in one launch
// The coefficient-gradient blocks (LDS- and matrix-core-bound) and the dx = t.N blocks (bound by the integer hash on the
// vector ALU) are independent once t, z and a zeroed dcoef exist, and lean on different units: launched as one grid, two
// blocks per compute unit, they overlap instead of queueing.  Both bodies use exactly 80 KB of LDS.
struct BwdParams {
    DcParams dc;
    TNParams tn;
    int dc_blocks;  // multiple of 8, so both parts keep their die assignment
};

__global__ __launch_bounds__(256, 2) void bwd_dc_tn_kernel(BwdParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    if ((int)blockIdx.x < p.dc_blocks)
        dc_block_direct(p.dc, lds, blockIdx.x);
    else
        tn_block(p.tn, lds, blockIdx.x - p.dc_blocks);
}

// ----------------------------------------------------------------------------------------------- the backward pass regrouped
// With room for the coefficient gradient's partial sums in the workspace nothing has to be zeroed first, so the two long
// contractions over dy, t = dy.C and dC = dy^T.z, can share a launch: both run the tile engine with four waves a block and
// wait on memory much of the time, and two blocks per compute unit fill each other's gaps (they also read the same dy).
// The second launch runs the dx = t.N blocks and, beside them, the blocks that add the partial sums up in split order.
struct BwdAParams {
    DcParams dc;
    DyCParams dyc;
    int dc_blocks;  // multiple of 8, so both parts keep their die assignment
};

__global__ __launch_bounds__(256, 2) void bwd_dc_dyc_kernel(BwdAParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    if ((int)blockIdx.x < p.dc_blocks) {
        dc_block_direct(p.dc, lds, blockIdx.x);
    } else {
        if (p.dyc.ctf && *p.dyc.ctf_flag)   // the forward pass left the transposed coefficients in the state
            dyc_block_direct(p.dyc, lds, blockIdx.x - p.dc_blocks);
        else
            dyc_block(p.dyc, lds, blockIdx.x - p.dc_blocks);
    }
}

struct BwdBParams {
    TNParams tn;
    RedParams red;
    int tn_blocks;
};

__global__ __launch_bounds__(256, 2) void bwd_tn_red_kernel(BwdBParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if ((int)blockIdx.x < p.tn_blocks)
        tn_block(p.tn, reinterpret_cast<bf16_t *>(smem_raw), blockIdx.x);
    else
        red_block(p.red, blockIdx.x - p.tn_blocks, gridDim.x - p.tn_blocks);
}

// dx = t . N for k <= 256 with t held in registers (rdb_stationary.hpp), alone and beside the reduction blocks.
template <int KG> __global__ __launch_bounds__(ST_THREADS, 1) void dx_tns_kernel(StParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    stationary_block<KG, false, true, true>(p, smem_raw, blockIdx.x);
}

struct BwdBsParams {
    StParams tn;
    RedParams red;
    int tn_blocks;
};

template <int KG> __global__ __launch_bounds__(ST_THREADS, 1) void bwd_tns_red_kernel(BwdBsParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if ((int)blockIdx.x < p.tn_blocks)
        stationary_block<KG, false, true, true>(p.tn, smem_raw, blockIdx.x);
    else
        red_block(p.red, blockIdx.x - p.tn_blocks, gridDim.x - p.tn_blocks);
}

// ----------------------------------------------------------------------------------------------- host side
void dc_params_from_state(DcParams &p, const void *state, const rdb_linear_desc *d);   // rdb_factored.hip

static bool dx_factored_ok(const rdb_linear_desc *d)
{
    return d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16 && d->coef_rows != 0 && d->k % 8 == 0 && d->in_f % 8 == 0 &&
           d->out_f % 8 == 0 && d->k > 0 && d->tokens > 0 && d->tokens < (1 << 30) && d->in_f < (1 << 30) && d->out_f < (1 << 30) &&
           d->k < (1 << 24) && d->tokens * d->k < (1ll << 29) && d->out_f * d->k < (1ll << 29);
}

// t = dy.C: [tokens x k] bf16, or, for the kernel that keeps t in registers, tokens padded to 32 and k to 64
int64_t linear_dx_factored_workspace(const rdb_linear_desc *d)
{
    if (!dx_factored_ok(d)) return 0;
    if (d->k <= ST_KMAX && cdiv(d->tokens, 32) * 32 * cdiv(d->k, 64) * 64 < (1ll << 29))
        return cdiv(d->tokens, 32) * 32 * cdiv(d->k, 64) * 64 * (int64_t)sizeof(bf16_t);
    return d->tokens * d->k * (int64_t)sizeof(bf16_t);
}

static int64_t align256(int64_t n) { return (n + 255) / 256 * 256; }

// Workspace of the regrouped backward pass: t, then the partial sums of the coefficient gradient.
// force_partial: also with a single token range (the call adds to dcoef instead of overwriting it).
int64_t linear_bwd_projected_workspace(const rdb_linear_desc *d, int num_cus, bool force_partial)
{
    if (!dx_factored_ok(d)) return 0;
    DcParams dc;
    make_dc_params(dc, nullptr, nullptr, d->out_f, d, num_cus);
    if (dc.splits == 1 && !force_partial) return linear_dx_factored_workspace(d);   // a single token range is stored straight into dcoef
    return align256(linear_dx_factored_workspace(d)) + (int64_t)dc.splits * d->out_f * d->k * (int64_t)sizeof(float);
}

static void make_dyc_params(DyCParams &p1, const void *dy, int64_t lddy, const void *coef, void *t, const rdb_linear_desc *d)
{
    p1.dy = (const bf16_t *)dy;
    p1.coef = (const bf16_t *)coef;
    p1.ctf = nullptr;
    p1.ctf_flag = nullptr;
    p1.osteps = 0;
    p1.kpad = 0;
    p1.t = (bf16_t *)t;
    p1.zero = nullptr;
    p1.zero_n = 0;
    p1.lddy = lddy;
    p1.tokens = (int)d->tokens;
    p1.out_f = (int)d->out_f;
    p1.k = (int)d->k;
    p1.tiles_c = (int)cdiv(d->k, K1_BC);
    p1.tiles_t = (int)cdiv(d->tokens, K1_BT);
    p1.frag_ksteps = 0;
}

// t . N with t in registers applies when k is short enough and dx fits a buffer descriptor.
static bool tn_stationary_ok(const rdb_linear_desc *d, int64_t lddx)
{   // dx and the padded, fragment-ordered t must each fit a buffer descriptor
    return d->k <= ST_KMAX && d->tokens * lddx < (1ll << 29) && cdiv(d->tokens, 32) * 32 * cdiv(d->k, 64) * 64 < (1ll << 29);
}

static int make_tns_params(StParams &q, void *dx, int64_t lddx, const void *t, const rdb_linear_desc *d, int num_cus)
{
    q.z = (const bf16_t *)t;
    q.coef = nullptr;
    q.bias = nullptr;
    q.y = (bf16_t *)dx;
    q.ldy = lddx;
    q.k = (int)d->k;
    q.seed = d->seed;
    return make_stationary_grid(q, d->tokens, d->in_f, num_cus);
}

// Returns RDB_E_UNSUPPORTED (without setting an error) when the request does not fit this algorithm.
int linear_dx_factored(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias,
                       const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!dx_factored_ok(d) || scale_bias) return RDB_E_UNSUPPORTED;  // the random-bias term is not low rank
    if (!workspace || workspace_bytes < linear_dx_factored_workspace(d) || ((uintptr_t)workspace & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens * lddy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    if (lddy % 8 || lddx % 8 || ((uintptr_t)dy & 15) || ((uintptr_t)coef & 15) || ((uintptr_t)dx & 15)) return RDB_E_UNSUPPORTED;
    // AUTO: up to 16 times the flops of one product on a stored W (the same bound as the forward's: see cheaper_factored there)
    if (d->algo == RDB_ALGO_AUTO && d->k * (d->in_f + d->out_f) >= 16 * d->in_f * d->out_f) return RDB_E_UNSUPPORTED;

    DyCParams p1;
    make_dyc_params(p1, dy, lddy, coef, workspace, d);
    const bool stationary = tn_stationary_ok(d, lddx);
    const int kg = (int)cdiv(d->k, 64);
    if (stationary) p1.frag_ksteps = kg * 4;
    int rc = launch_engine(dx_dyc_kernel, p1, p1.tiles_c * p1.tiles_t, engine_smem<K1_BC, K1_BT, X_BK, M_CONT, K_CONT>(), s, "dx_dyc_kernel");
    if (rc) return rc;
    if (stationary) {
        StParams q;
        const int items = make_tns_params(q, dx, lddx, workspace, d, num_cus);
        const size_t smem = stationary_smem(kg);
        switch (kg) {
        case 1: return launch_stationary(dx_tns_kernel<1>, q, items, smem, s, "dx_tns_kernel<1>");
        case 2: return launch_stationary(dx_tns_kernel<2>, q, items, smem, s, "dx_tns_kernel<2>");
        case 3: return launch_stationary(dx_tns_kernel<3>, q, items, smem, s, "dx_tns_kernel<3>");
        default: return launch_stationary(dx_tns_kernel<4>, q, items, smem, s, "dx_tns_kernel<4>");
        }
    }
    TNParams p2;
    const int items = make_tn_params(p2, dx, lddx, workspace, d);
    return launch_engine(dx_tn_kernel, p2, items, engine_smem<K2_BI, K2_BT, X_BK, K_CONT, K_CONT>(), s, "dx_tn_kernel");
}

// Which of the two launches linear_bwd_projected enqueues: bit 0 the first, bit 1 the second (3: both).  Timing tools launch one
// of them alone (rdb_linear_bwd_projected_part); the mask is the calling thread's.
static thread_local int g_bwd_parts = 3;
void set_bwd_projected_parts(int mask) { g_bwd_parts = mask & 3; }

// Whole backward pass of the layer from the saved projection z: dx = (dy.C).N and dcoef = dy^T.z in two launches.
// Returns RDB_E_UNSUPPORTED (without setting an error) when the request does not fit.
// accumulate: dcoef += instead of dcoef = (a later chunk of tokens of a layer whose activations are passed in chunks).
// dc_bf16: dcoef is bf16 [out_f x k], the fp32 sums rounded once by the blocks that add them up (needs the workspace with room
// for the sums, linear_bwd_projected_workspace(d, num_cus, true), and is not combined with accumulate).
int linear_bwd_projected(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *z, const void *coef,
                         const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, bool accumulate, bool dc_bf16,
                         hipStream_t s)
{
    if (!dx_factored_ok(d)) return RDB_E_UNSUPPORTED;
    if (dc_bf16 && (accumulate || workspace_bytes < linear_bwd_projected_workspace(d, num_cus, true))) return RDB_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < linear_dx_factored_workspace(d) || ((uintptr_t)workspace & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens * lddy >= (1ll << 29) || lddy % 8 || lddx % 8) return RDB_E_UNSUPPORTED;
    if (((uintptr_t)dy & 15) || ((uintptr_t)coef & 15) || ((uintptr_t)dx & 15) || ((uintptr_t)z & 15) || ((uintptr_t)dcoef & 15))
        return RDB_E_UNSUPPORTED;
    DyCParams p1;
    make_dyc_params(p1, dy, lddy, coef, workspace, d);
    const size_t smem_dc = engine_smem<KD_BO, KD_BM, X_BK, M_CONT, M_CONT>(), smem_tn = engine_smem<K2_BI, K2_BT, X_BK, K_CONT, K_CONT>();
    const size_t smem_dyc = engine_smem<K1_BC, K1_BT, X_BK, M_CONT, K_CONT>();
    if (workspace_bytes >= linear_bwd_projected_workspace(d, num_cus, accumulate || dc_bf16)) {
        BwdAParams a;
        const int dc_items = make_dc_params(a.dc, dcoef, dy, lddy, d, num_cus);
        dc_params_from_state(a.dc, z, d);
        // one token range only: its sums are the result, stored straight into dcoef, and nothing is left to add up
        const bool direct = a.dc.splits == 1 && !accumulate && !dc_bf16;
        a.dc.partial = direct ? dcoef : reinterpret_cast<float *>(static_cast<char *>(workspace) + align256(linear_dx_factored_workspace(d)));
        a.dyc = p1;
        {   // the transposed coefficients, if the forward pass left them in the state (its header says so)
            const ProjLayout L = proj_layout(d);
            a.dyc.ctf = reinterpret_cast<const bf16_t *>(static_cast<const char *>(z) + L.ctf_off);
            a.dyc.ctf_flag = static_cast<const uint32_t *>(z);
            a.dyc.osteps = (int)(L.out64 / 16);
            a.dyc.kpad = L.kpad;
        }
        if (tn_stationary_ok(d, lddx)) a.dyc.frag_ksteps = (int)cdiv(d->k, 64) * 4;   // the t.N kernel below keeps t in registers
        a.dc_blocks = xcd_grid_size(dc_items);
        int rc = RDB_OK, red_splits = a.dc.splits;
        if (!(g_bwd_parts & 1)) {
            if (big_bwd_applies(d, num_cus) && !a.dyc.frag_ksteps) red_splits = 1;
        } else if (big_bwd_applies(d, num_cus) && !a.dyc.frag_ksteps) {
            // long coefficient dimension and many tiles: both products on 256-wide tiles; a dC tile contracts all tokens, so
            // there is one set of sums, stored where the first split's would go
            rc = linear_bwd_big(workspace, a.dc.partial, dy, lddy, z, coef, d, num_cus, true, true, s);
            red_splits = 1;
        } else {
            size_t smem = smem_dc > smem_dyc ? smem_dc : smem_dyc;
            if (int rl = reserve_lds(reinterpret_cast<const void *>(bwd_dc_dyc_kernel), smem, "bwd_dc_dyc_kernel")) return rl;
            bwd_dc_dyc_kernel<<<a.dc_blocks + xcd_grid_size(p1.tiles_c * p1.tiles_t), 256, smem, s>>>(a);
            rc = check_launch("bwd_dc_dyc_kernel");
        }
        if (rc) return rc;
        if (!(g_bwd_parts & 2)) return RDB_OK;
        RedParams red;
        red.partial = a.dc.partial;
        red.out = dcoef;
        red.n = d->out_f * d->k;
        red.splits = red_splits;
        red.accumulate = accumulate ? 1 : 0;
        red.out_bf16 = dc_bf16 ? 1 : 0;
        if (tn_stationary_ok(d, lddx)) {
            BwdBsParams bs;
            const int items = make_tns_params(bs.tn, dx, lddx, workspace, d, num_cus);
            bs.red = red;
            bs.tn_blocks = xcd_grid_size(items);
            int rblocks = (int)cdiv(red.n / 4 * red.splits, ST_THREADS * 16);   // about 16 loads of 16 bytes a thread
            if (rblocks > num_cus / 2) rblocks = num_cus / 2;
            // a block of this kernel has a compute unit to itself: where the product's blocks leave units free, no more reduction
            // blocks than those, so that the launch is one round of blocks
            if (bs.tn_blocks < num_cus && rblocks > num_cus - bs.tn_blocks) rblocks = num_cus - bs.tn_blocks;
            if (rblocks < 1) rblocks = 1;
            if (direct) rblocks = 0;
            const int kg = (int)cdiv(d->k, 64);
            const size_t smem_s = stationary_smem(kg);
            const void *fn = kg == 1 ? (const void *)bwd_tns_red_kernel<1> : kg == 2 ? (const void *)bwd_tns_red_kernel<2>
                           : kg == 3 ? (const void *)bwd_tns_red_kernel<3> : (const void *)bwd_tns_red_kernel<4>;
            if (int rl = reserve_lds(fn, smem_s, "bwd_tns_red_kernel")) return rl;
            const dim3 grid(bs.tn_blocks + rblocks), block(ST_THREADS);
            switch (kg) {
            case 1: bwd_tns_red_kernel<1><<<grid, block, smem_s, s>>>(bs); break;
            case 2: bwd_tns_red_kernel<2><<<grid, block, smem_s, s>>>(bs); break;
            case 3: bwd_tns_red_kernel<3><<<grid, block, smem_s, s>>>(bs); break;
            default: bwd_tns_red_kernel<4><<<grid, block, smem_s, s>>>(bs); break;
            }
            return check_launch("bwd_tns_red_kernel");
        }
        BwdBParams b;
        const int tn_items = make_tn_params(b.tn, dx, lddx, workspace, d);
        b.tn_blocks = xcd_grid_size(tn_items);
        b.red = red;
        int red_blocks = (int)cdiv(b.red.n / 4 * b.red.splits, 256 * 16);
        if (red_blocks > num_cus) red_blocks = num_cus;
        if (red_blocks < 1) red_blocks = 1;
        if (direct) red_blocks = 0;
        if (int rl = reserve_lds(reinterpret_cast<const void *>(bwd_tn_red_kernel), smem_tn, "bwd_tn_red_kernel")) return rl;
        bwd_tn_red_kernel<<<b.tn_blocks + red_blocks, 256, smem_tn, s>>>(b);
        return check_launch("bwd_tn_red_kernel");
    }
    // workspace for t only: dy.C first (clearing dcoef on the side), then the coefficient gradient with atomics beside t.N
    p1.zero = accumulate ? nullptr : dcoef;
    p1.zero_n = d->out_f * d->k;
    int rc = launch_engine(dx_dyc_kernel, p1, p1.tiles_c * p1.tiles_t, smem_dyc, s, "dx_dyc_kernel");
    if (rc) return rc;
    BwdParams p;
    const int dc_items = make_dc_params(p.dc, dcoef, dy, lddy, d, num_cus);
    dc_params_from_state(p.dc, z, d);
    const int tn_items = make_tn_params(p.tn, dx, lddx, workspace, d);
    p.dc_blocks = xcd_grid_size(dc_items);
    const size_t smem = smem_dc > smem_tn ? smem_dc : smem_tn;
    if (int rl = reserve_lds(reinterpret_cast<const void *>(bwd_dc_tn_kernel), smem, "bwd_dc_tn_kernel")) return rl;
    bwd_dc_tn_kernel<<<p.dc_blocks + xcd_grid_size(tn_items), 256, smem, s>>>(p);
    return check_launch("bwd_dc_tn_kernel");
}

}  // namespace rdb
