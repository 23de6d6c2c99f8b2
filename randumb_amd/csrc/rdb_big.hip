// The factored algorithm's dense products on 256-wide tiles, for layers with a long coefficient dimension (k > 256) and
// enough tiles to give every compute unit one:
//   big_y_kernel    y[tok, o]  = sum_m z[tok, m] * C[o, m] (+ bias[o])          256 (o) x 256 (tok) tiles
//   big_bwd_kernel  t[tok, m]  = sum_o dy[tok, o] * C[o, m]                       256 (m) x 128 (tok) tiles, and in the same launch
//                   dC[o, m]   = sum_tok dy[tok, o] * z[tok, m]                   256 (o) x 256 (m) tiles over all tokens
// z, z^T and C^T come from the projection state in fragment order (rdb_direct.hpp: ProjLayout).  One persistent block per
// compute unit (rdb_big.hpp).  Replaces materialize() + dense product and MmBackward's two products
// (src/rten_cpp/RandumbTensor.py:942-946, 979-990) for such layers, as the 128-wide kernels of rdb_factored.hip / rdb_dx.hip do
// for all others.
#include "rdb_big.hpp"
#include "rdb_blocks.hpp"
#include <atomic>
#include <type_traits>

namespace rdb {

constexpr int BG = 256;   // tile edge

// Work item w of the forward product -> (output tile, token tile).  Neighbouring items run at the same time on one die: they
// are numbered so that 32 of them cover 8 output tiles x 4 token tiles (6 MB of operands, which a die's L2 holds) rather
// than 32 x 1 (16.5 MB): groups of 4 token tiles, walked through output tile by output tile.
constexpr int BY_GROUP_T = 4;
__device__ __forceinline__ void big_y_decode(int w, int tiles_o, int tiles_t, int &to, int &tt)
{
    const int per_group = BY_GROUP_T * tiles_o, group = w / per_group, in_group = w - group * per_group;
    const int first_t = group * BY_GROUP_T, gsize = tiles_t - first_t < BY_GROUP_T ? tiles_t - first_t : BY_GROUP_T;
    to = in_group / gsize;
    tt = first_t + in_group - to * gsize;
}

// 0: never use these kernels, 1: when the layer has enough tiles (default), 2: whenever the shapes allow (tests)
static std::atomic<int> g_big_mode{1};
void set_big_tiles_mode(int mode) { g_big_mode.store(mode < 0 ? 0 : mode > 2 ? 2 : mode); }
int big_tiles_mode() { return g_big_mode.load(); }

static bool enough_tiles(int64_t tiles, int num_cus)
{
    const int mode = g_big_mode.load();
    return mode == 2 || (mode == 1 && tiles * 2 >= num_cus);
}

// ----------------------------------------------------------------------------------------------- y = z . C^T
struct BigYParams {
    const bf16_t *zf;   // fragment order, rows = tokens (tok32 / 32 row blocks), kpad / 16 k-steps
    const bf16_t *coef;
    const bf16_t *bias;
    bf16_t *y;
    int64_t ldy, y_elems;
    int tokens, out_f, k, kpad, tok32;
    int tiles_o, tiles_t;
};

// Tiles are dealt out in rounds of one per block.  A last round that would occupy at most half of the blocks is dealt out as
// half tiles (256 output features x 128 tokens) instead, two blocks to a tile, so that no block idles through a whole tile.
constexpr int BY_HALF = 128;

template <bool BIAS> __global__ __launch_bounds__(256, 1) void big_y_kernel(BigYParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    typedef GlobalOperand<BG, 64, K_CONT> PA;   // C: rows = output features
    typedef FragOperand<BG, 64> PB;             // z: rows = tokens
    typedef FragOperand<BY_HALF, 64> PH;        // z: the tokens of a half tile
    const int total = p.tiles_o * p.tiles_t, vtotal = (total + 7) / 8 * 8, nblk = gridDim.x, nstage = (p.k + 63) / 64;
    const int full_rounds = vtotal / nblk, rest = vtotal - full_rounds * nblk;
    const bool halves = rest > 0 && 2 * rest <= nblk;
    const int my_rounds = full_rounds + ((!halves && (int)blockIdx.x < rest) ? 1 : 0);
    // this block's r-th tile: virtual index v -> work item w (a die's items are neighbours: they share z tiles and C)
    int r = 0;
#ifdef RDB_STAMPS
    int rdb_stamp_seq = 0;   // a timing harness records the block's tiles one after the other
#endif
    auto next = [&]() {
        for (; r < my_rounds; ++r) {
            const int w = xcd_work_item(r * nblk + (int)blockIdx.x, total);
            if (w < total) { ++r; return w; }
        }
        return -1;
    };
    PA pa;
    auto init_a = [&](int to) { pa = PA{p.coef, (int64_t)p.k, to * BG, p.out_f, p.k, (int64_t)p.out_f * p.k}; };
    int w = next();
    if (w >= 0) {
        PB pb;
        BigRegs<PA, PB> regs;
        auto request = [&](int w) {
            int to, tt;
            big_y_decode(w, p.tiles_o, p.tiles_t, to, tt);
            init_a(to);
            pb.src = p.zf;
            pb.ksteps = p.kpad >> 4;
            pb.nrb = p.tok32 >> 5;
            pb.rb0 = tt * (BG / 32);
            pb.klim_steps = p.kpad >> 4;
            big_prefetch(regs, pa, pb, 0);
        };
        request(w);
        while (true) {
            int to, tt;
            big_y_decode(w, p.tiles_o, p.tiles_t, to, tt);
            const int o0 = to * BG, tok0 = tt * BG;
            f32x16 acc[BG / 64][BG / 64];
            RDB_STAMP(0);
            big_zero<BG, BG>(acc);
            big_mainloop<BG, BG>(acc, lds, regs, pa, pb, nstage);
            RDB_STAMP(1);
            BigBias<BG> bias;   // requested ahead of the next tile's first stages, which the epilogue does not wait for
            if (BIAS) big_load_bias<BG>(bias, p.bias, o0, p.out_f);
            const int wn = next();
            if (wn >= 0) request(wn);   // on its way while this tile leaves
            __builtin_amdgcn_sched_barrier(0);
            RDB_STAMP(2);
            big_store_bf16<BG, BG, BIAS, true>(acc, lds, p.y, p.ldy, p.y_elems, o0, p.out_f, tok0, p.tokens, bias, opaque_tid());
            RDB_STAMP(3);
#ifdef RDB_STAMPS
            ++rdb_stamp_seq;
#endif
            if (wn < 0) break;
            w = wn;
        }
    }
    if (!halves || (int)blockIdx.x >= 2 * rest) return;
    w = xcd_work_item(full_rounds * nblk + ((int)blockIdx.x >> 1), total);
    if (w >= total) return;
    {
        int to, tt;
        big_y_decode(w, p.tiles_o, p.tiles_t, to, tt);
        const int o0 = to * BG, tok0 = tt * BG + ((int)blockIdx.x & 1) * BY_HALF;
        PH pb;
        BigRegs<PA, PH> regs;
        init_a(to);
        pb.src = p.zf;
        pb.ksteps = p.kpad >> 4;
        pb.nrb = p.tok32 >> 5;
        pb.rb0 = tok0 >> 5;
        pb.klim_steps = p.kpad >> 4;
        big_prefetch(regs, pa, pb, 0);
        f32x16 acc[BG / 64][BY_HALF / 64];
        big_zero<BG, BY_HALF>(acc);
        RDB_STAMP(0);
        big_mainloop<BG, BY_HALF>(acc, lds, regs, pa, pb, nstage);
        RDB_STAMP(1);
        BigBias<BG> bias;
        if (BIAS) big_load_bias<BG>(bias, p.bias, o0, p.out_f);
        RDB_STAMP(2);
        big_store_bf16<BG, BY_HALF, BIAS, true>(acc, lds, p.y, p.ldy, p.y_elems, o0, p.out_f, tok0, p.tokens, bias, opaque_tid());
        RDB_STAMP(3);
    }
}

// ----------------------------------------------------------------------------------------------- t = dy . C and dC = dy^T . z
constexpr int BT_TOK = 128;   // token edge of a t tile

struct BigBwdParams {
    const bf16_t *dy;
    int64_t lddy;
    const bf16_t *coef;
    const bf16_t *ctf;            // C transposed in fragment order (rows = coefficients), valid when *ctf_flag != 0
    const uint32_t *ctf_flag;
    const bf16_t *ztf;            // z transposed in fragment order (rows = coefficients)
    bf16_t *t;                    // [tokens x k] row-major
    float *dc;                    // [out_f x k]: dcoef itself, or the partial-sum area a reduction adds to dcoef
    int tokens, out_f, k, kpad;
    int osteps, tsteps;           // k-steps per row block of ctf (out_f rounded up to 64, / 16) and of ztf (tokens likewise)
    int t_tiles_m, t_tiles_t;     // t tiles: 256 coefficients x 128 tokens; 0 tiles: the launch computes dC only
    int c_tiles_o, c_tiles_m;     // dC tiles: 256 output features x 256 coefficients; 0 tiles: t only
    int t_first;                  // the t tiles come first in the list (they are the longer ones), else the dC tiles
};

// t tiles of one block.  CT: C^T from its fragment-ordered copy; otherwise C itself, staged as an M_CONT operand.
template <bool CT> __device__ __forceinline__ void big_t_items(const BigBwdParams &p, bf16_t *lds, int &r, int base, int n1)
{
    const int n1v = (n1 + 7) / 8 * 8;
    typedef typename std::conditional<CT, FragOperand<BG, 64>, GlobalOperand<BG, 64, M_CONT>>::type PA;   // rows = coefficients
    typedef GlobalOperand<BT_TOK, 64, K_CONT> PB;                                                          // dy: rows = tokens
    const int nblk = gridDim.x, nstage = (p.out_f + 63) / 64;
    auto next = [&]() {
        for (;; ++r) {
            const int v = big_item(blockIdx.x, r, nblk) - base;
            if (v >= n1v) return -1;   // r stays at the first round past the t tiles
            const int w = xcd_work_item(v, n1);
            if (w < n1) { ++r; return w; }
        }
    };
    PA pa;
    PB pb;
    BigRegs<PA, PB> regs;
    auto request = [&](int w) {
        const int m0 = (w % p.t_tiles_m) * BG, tok0 = (w / p.t_tiles_m) * BT_TOK;
        if constexpr (CT) {
            pa.src = p.ctf;
            pa.ksteps = p.osteps;
            pa.nrb = p.kpad >> 5;
            pa.rb0 = m0 >> 5;
            pa.klim_steps = p.osteps;
        } else {
            pa = PA{p.coef, (int64_t)p.k, m0, p.k, p.out_f, (int64_t)p.out_f * p.k};
        }
        pb = PB{p.dy, p.lddy, tok0, p.tokens, p.out_f, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
        big_prefetch(regs, pa, pb, 0);
    };
    int w = next();
    if (w < 0) return;
    request(w);
    while (true) {
        const int m0 = (w % p.t_tiles_m) * BG, tok0 = (w / p.t_tiles_m) * BT_TOK;
        f32x16 acc[BG / 64][BT_TOK / 64];
        big_zero<BG, BT_TOK>(acc);
        big_mainloop<BG, BT_TOK>(acc, lds, regs, pa, pb, nstage);
        const int wn = next();
        if (wn >= 0) request(wn);
        __builtin_amdgcn_sched_barrier(0);
        big_store_bf16<BG, BT_TOK, false>(acc, lds, p.t, p.k, (int64_t)p.tokens * p.k, m0, p.k, tok0, p.tokens, BigBias<BG>(), opaque_tid());
        if (wn < 0) break;
        w = wn;
    }
}

// dC tiles of one block, from the block's round r on; `base`: index of the first dC tile in the launch's list.
__device__ __forceinline__ void big_dc_items(const BigBwdParams &p, bf16_t *lds, int &r, int base, int n2)
{
    typedef GlobalOperand<BG, 64, M_CONT> PA;   // dy: rows = output features, contraction = tokens
    typedef FragOperand<BG, 64> PB;             // z^T: rows = coefficients
    const int nblk = gridDim.x, nstage = (p.tokens + 63) / 64, n2v = (n2 + 7) / 8 * 8;
    auto next = [&]() {
        for (;; ++r) {
            const int v = big_item(blockIdx.x, r, nblk) - base;
            if (v >= n2v) return -1;
            const int w = xcd_work_item(v, n2);
            if (w < n2) { ++r; return w; }
        }
    };
    PA pa;
    PB pb;
    BigRegs<PA, PB> regs;
    auto request = [&](int w) {
        pa = PA{p.dy, p.lddy, (w / p.c_tiles_m) * BG, p.out_f, p.tokens, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
        pb.src = p.ztf;
        pb.ksteps = p.tsteps;
        pb.nrb = p.kpad >> 5;
        pb.rb0 = (w % p.c_tiles_m) * (BG / 32);
        pb.klim_steps = p.tsteps;
        big_prefetch(regs, pa, pb, 0);
    };
    int w = next();
    if (w < 0) return;
    request(w);
    while (true) {
        const int m0 = (w % p.c_tiles_m) * BG, o0 = (w / p.c_tiles_m) * BG;
        f32x16 acc[BG / 64][BG / 64];
        big_zero<BG, BG>(acc);
        big_mainloop<BG, BG>(acc, lds, regs, pa, pb, nstage);
        const int wn = next();
        if (wn >= 0) request(wn);
        __builtin_amdgcn_sched_barrier(0);
        big_store_f32<BG, BG>(acc, lds, p.dc, p.k, (int64_t)p.out_f * p.k, o0, p.out_f, m0, p.k, opaque_tid());
        if (wn < 0) break;
        w = wn;
    }
}

// The launch's list holds the tiles of the longer kind first (a t tile contracts out_f with half-size stages, a dC tile the
// tokens) and is dealt out to the blocks in rows of alternating direction (big_item): the blocks that got a long tile in
// one row get the later, shorter ones of the next.  A block's rounds walk through the list in order, so it finishes its
// tiles of the first kind before it starts on the second.
__global__ __launch_bounds__(256, 1) void big_bwd_kernel(BigBwdParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    const int n1 = p.t_tiles_m * p.t_tiles_t, n1v = (n1 + 7) / 8 * 8, n2 = p.c_tiles_o * p.c_tiles_m, n2v = (n2 + 7) / 8 * 8;
    const bool ct = n1 && p.ctf && *p.ctf_flag;
    int r = 0;
    if (p.t_first) {
        if (n1) {
            if (ct) big_t_items<true>(p, lds, r, 0, n1);
            else big_t_items<false>(p, lds, r, 0, n1);
        }
        if (n2) big_dc_items(p, lds, r, n1v, n2);
    } else {
        if (n2) big_dc_items(p, lds, r, 0, n2);
        if (n1) {
            if (ct) big_t_items<true>(p, lds, r, n2v, n1);
            else big_t_items<false>(p, lds, r, n2v, n1);
        }
    }
}

// ----------------------------------------------------------------------------------------------- host side
static bool big_aligned16(const void *q) { return ((uintptr_t)q & 15) == 0; }

// Do these kernels apply to the layer's forward product / backward pass?  (The shape conditions of the 128-wide kernels are
// checked by the callers, which fall back to those kernels when the answer is no.)
bool big_fwd_applies(const rdb_linear_desc *d, int num_cus)
{
    const ProjLayout L = proj_layout(d);
    return L.ok && !L.fits_regs && enough_tiles(cdiv(d->out_f, BG) * cdiv(d->tokens, BG), num_cus);
}
bool big_bwd_applies(const rdb_linear_desc *d, int num_cus)
{
    const ProjLayout L = proj_layout(d);
    // every dC tile contracts all tokens (no partial sums over token ranges), so the tiles alone must fill the chip; and the t
    // tiles, each of which contracts all of out_f, must not be so few that a handful of blocks is left with all of that work
    return L.ok && !L.fits_regs && enough_tiles(cdiv(d->out_f, BG) * cdiv(d->k, BG), num_cus) &&
           enough_tiles(2 * cdiv(d->k, BG) * cdiv(d->tokens, BT_TOK), num_cus);
}

template <class K, class P> static int launch_big(K kernel, const P &p, int items, int num_cus, size_t smem, hipStream_t s, const char *name)
{
    if (int rl = reserve_lds(reinterpret_cast<const void *>(kernel), smem, name)) return rl;
    int blocks = num_cus / 8 * 8;   // a multiple of 8: a block's tiles stay on one die's share of the list
    if (blocks < 8) blocks = 8;
    const int vitems = (items + 7) / 8 * 8;
    if (blocks > vitems) blocks = vitems;
    kernel<<<blocks, 256, smem, s>>>(p);
    return check_launch(name);
}

int linear_fwd_big(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    const ProjLayout L = proj_layout(d);
    if (!L.ok || d->coef_dtype != RDB_BF16 || ldy % 8 || !big_aligned16(y) || !big_aligned16(state) || !big_aligned16(coef)) return RDB_E_UNSUPPORTED;
    if (((uintptr_t)bias & 7) || d->tokens * ldy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    BigYParams p;
    p.zf = reinterpret_cast<const bf16_t *>(static_cast<const char *>(state) + L.zf_off);
    p.coef = (const bf16_t *)coef;
    p.bias = (const bf16_t *)bias;
    p.y = (bf16_t *)y;
    p.ldy = ldy;
    p.y_elems = (d->tokens - 1) * ldy + d->out_f;
    p.tokens = (int)d->tokens;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.kpad = L.kpad;
    p.tok32 = (int)L.tok32;
    p.tiles_o = (int)cdiv(d->out_f, BG);
    p.tiles_t = (int)cdiv(d->tokens, BG);
    typedef OperandTile<BG, 64, K_CONT> TA;
    typedef FragTile<BG, 64> TB;
    if (bias) return launch_big(big_y_kernel<true>, p, p.tiles_o * p.tiles_t, num_cus, big_smem<BG, BG, TA, TB>(), s, "big_y_kernel<bias>");
    return launch_big(big_y_kernel<false>, p, p.tiles_o * p.tiles_t, num_cus, big_smem<BG, BG, TA, TB>(), s, "big_y_kernel");
}

// First launch of the backward pass: t (row-major, for the t . N kernel of the tile engine) and dC.  `dc`: where the
// coefficient gradient's sums go (dcoef, or the area a reduction adds to dcoef).  want_t / want_dc: which of the two
// (t alone needs no state, dC alone no coefficients).
int linear_bwd_big(void *t, float *dc, const void *dy, int64_t lddy, const void *state, const void *coef, const rdb_linear_desc *d, int num_cus,
                   bool want_t, bool want_dc, hipStream_t s)
{
    const ProjLayout L = proj_layout(d);
    if (!L.ok || d->tokens * lddy >= (1ll << 29) || lddy % 8) return RDB_E_UNSUPPORTED;
    if ((want_t && (d->coef_dtype != RDB_BF16 || !coef || !t)) || (want_dc && (!state || !dc))) return RDB_E_UNSUPPORTED;
    if (!big_aligned16(dy) || !big_aligned16(state) || !big_aligned16(coef) || !big_aligned16(t) || !big_aligned16(dc)) return RDB_E_UNSUPPORTED;
    BigBwdParams p;
    p.dy = (const bf16_t *)dy;
    p.lddy = lddy;
    p.coef = (const bf16_t *)coef;
    // without a state (the input gradient called on its own) C is staged from its row-major form
    p.ctf = state ? reinterpret_cast<const bf16_t *>(static_cast<const char *>(state) + L.ctf_off) : nullptr;
    p.ctf_flag = static_cast<const uint32_t *>(state);
    p.ztf = state ? reinterpret_cast<const bf16_t *>(static_cast<const char *>(state) + L.ztf_off) : nullptr;
    p.t = (bf16_t *)t;
    p.dc = dc;
    p.tokens = (int)d->tokens;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.kpad = L.kpad;
    p.osteps = (int)(L.out64 / 16);
    p.tsteps = (int)(L.tok64 / 16);
    p.t_tiles_m = want_t ? (int)cdiv(d->k, BG) : 0;
    p.t_tiles_t = want_t ? (int)cdiv(d->tokens, BT_TOK) : 0;
    p.c_tiles_o = want_dc ? (int)cdiv(d->out_f, BG) : 0;
    p.c_tiles_m = want_dc ? (int)cdiv(d->k, BG) : 0;
    typedef OperandTile<BG, 64, M_CONT> TM;
    typedef FragTile<BG, 64> TF;
    typedef OperandTile<BT_TOK, 64, K_CONT> TD;
    constexpr size_t smem_dc = big_smem<BG, BG, TM, TF>(), smem_t = big_smem<BG, BT_TOK, TM, TD>();
    p.t_first = d->out_f >= 2 * d->tokens;   // stages of 64 at half the matrix work against stages of 64 over the tokens
    const int items = (p.t_tiles_m * p.t_tiles_t + 7) / 8 * 8 + (p.c_tiles_o * p.c_tiles_m + 7) / 8 * 8;
    return launch_big(big_bwd_kernel, p, items, num_cus, smem_dc > smem_t ? smem_dc : smem_t, s, "big_bwd_kernel");
}

}  // namespace rdb
