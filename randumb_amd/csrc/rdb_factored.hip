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
#include <algorithm>

namespace rdb {

constexpr float INV_2_31 = 4.656612873077392578125e-10f;
constexpr int F_BK = 64;

// ----------------------------------------------------------------------------------------------- z = x . N^T
// tile: 32 coefficients (hashed) x 256 tokens, contraction over in_f.  The noise tile is hashed once per block, so the hash
// work of the kernel is (tokens / 256) * in_f * k: the token tile is long and the coefficient tile short.
constexpr int KZ_BM = 32, KZ_BT = 256;

struct ZParams {
    const bf16_t *x;
    const bf16_t *coef;  // NULL, or C [out_f x k] to transpose into ctf on the side
    bf16_t *zf;          // z for the forward product: fragment order, rows = tokens
    bf16_t *ztf;         // z transposed in fragment order, rows = coefficients
    bf16_t *ctf;         // C transposed in fragment order, rows = coefficients
    uint32_t *flag;      // header word 0 of the state: 1 when ctf has been written by this launch
    int64_t ldx;
    int tokens, in_f, out_f, k;
    int kpad, tok32, tok64, out64;
    int tiles_m, tiles_t;
    uint32_t seed;
    unsigned long long *sync;   // NULL, or slots [tiles_t][tiles_m + 1]: a block sets its slot to sync_tag when its tile is in memory;
                                // slot tiles_m of a token tile counts its consumers and is cleared by the block of coefficient tile 0
    unsigned long long sync_tag;
};

// Eight waves, two to a SIMD: the tile's noise is hashed once per stage by all 512 threads (4 values each) on the vector ALU,
// and while one wave of a SIMD hashes or waits for its x pieces the other one's MFMAs run.  Per stage of 64 input features:
// x pieces (loaded two stages ahead) and the next stage's noise go registers -> LDS, 4 MFMAs per wave (its 32 tokens), one
// barrier.  Written without the 256-thread tile engine; the LDS layouts and fragment reads are the engine's (OperandTile).
constexpr int KZ_THREADS = 512;

// `block` of `nblocks`: index of this block among the blocks that run this body; all KZ_THREADS threads must call.
__device__ __forceinline__ void z_block(const ZParams &p, unsigned char *smem_raw, int block, int nblocks)
{
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    if (block == 0 && t == 0) {
        p.flag[0] = p.coef ? 1u : 0u;
        p.flag[1] = 0u;   // nobody has given up waiting on this state
    }
    // C transposed into fragment order, a 1 KB unit (32 coefficients x 16 output features) per wave and turn: lane (r, g)
    // gathers C[o0 + 8 g + j][m0 + r], j = 0..7 (32 lanes read 64 consecutive bytes of a row) and stores its 16 bytes.
    // The first turn's loads are issued here and stored after the tile's main loop, which hides their latency.
    const int osteps = p.out64 >> 4, units = p.coef ? (p.kpad >> 5) * osteps : 0;
    auto gather_unit = [&](int u, uint32_t (&w)[8]) {   // the raw values: combining them would wait for the loads
        const int mb = u / osteps, os = u % osteps, m = mb * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int o = os * 16 + (lane >> 5) * 8 + j;
            w[j] = (m < p.k && o < p.out_f) ? p.coef[(int64_t)o * p.k + m] : 0u;
        }
    };
    auto store_unit = [&](int u, const uint32_t (&w)[8]) {
        const i32x4 v = {(int)(w[0] | (w[1] << 16)), (int)(w[2] | (w[3] << 16)), (int)(w[4] | (w[5] << 16)), (int)(w[6] | (w[7] << 16))};
        store_stream(reinterpret_cast<i32x4 *>(p.ctf + (int64_t)u * 512 + lane * 8), v);
    };
    const int unit0 = block * (KZ_THREADS / 64) + wave, unit_step = nblocks * (KZ_THREADS / 64);
    uint32_t cw0[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    if (unit0 < units) gather_unit(unit0, cw0);
    auto finish_units = [&]() {
        if (unit0 < units) store_unit(unit0, cw0);
        for (int u = unit0 + unit_step; u < units; u += unit_step) {
            uint32_t w[8];
            gather_unit(u, w);
            store_unit(u, w);
        }
    };
    // work item = (token tile, coefficient tile), coefficient tile fastest: neighbours share the x tile
    const int w = xcd_work_item(block, p.tiles_m * p.tiles_t);
    if (w >= p.tiles_m * p.tiles_t) {
        finish_units();
        return;
    }
    const int m0 = (w % p.tiles_m) * KZ_BM, tok0 = (w / p.tiles_m) * KZ_BT;
    // A replay of a recorded launch carries the tag it was recorded with.  The consumers clear the slots when all of them are
    // past their wait; should one of them have given up in an earlier replay, a slot may still hold the tag: take it back
    // before this tile is touched.
    if (p.sync && t == 0)
        __hip_atomic_store(p.sync + (int64_t)(w / p.tiles_m) * (p.tiles_m + 1) + w % p.tiles_m, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    RDB_STAMP(0);
    typedef OperandTile<KZ_BM, F_BK, K_CONT> TN;   // noise tile: rows = coefficients, contraction = input features
    typedef OperandTile<KZ_BT, F_BK, K_CONT> TX;   // x tile: rows = tokens
    constexpr int STAGE = TN::LDS_ELEMS + TX::LDS_ELEMS, XP = KZ_BT * F_BK / 8 / KZ_THREADS;   // x pieces per thread and stage: 4
    const int nstage = (p.in_f + F_BK - 1) / F_BK;
    const __amdgpu_buffer_rsrc_t rs_x =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.x), 0, (int)(((int64_t)(p.tokens - 1) * p.ldx + p.in_f) * 2), 0x00020000);
    // this thread's x pieces: rows idx / 8, 16-byte chunk idx % 8 of the stage's 64 features
    uint32_t xoff[XP];
    int xlds[XP];
#pragma unroll
    for (int q = 0; q < XP; ++q) {
        const int idx = q * KZ_THREADS + t, row = idx >> 3, c = idx & 7;
        xoff[q] = (tok0 + row < p.tokens) ? (uint32_t)(((int64_t)(tok0 + row) * p.ldx + c * 8) * 2) : BUFFER_OOB;
        xlds[q] = row * TX::LD + ((c ^ TX::swz(row)) * 8);
    }
    const int xc8 = (t & 7) * 8;   // the same for all of a thread's pieces (512 % 8 == 0)
    auto load_x = [&](f32x4 (&r)[XP], int stage) {
        const uint32_t adv = (stage * F_BK + xc8 < p.in_f) ? (uint32_t)(stage * F_BK * 2) : BUFFER_OOB;   // in_f % 8 == 0
#pragma unroll
        for (int q = 0; q < XP; ++q) r[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_x, (int)(xoff[q] + adv), 0, 0));
    };
    auto store_x = [&](bf16_t *buf, const f32x4 (&r)[XP]) {
#pragma unroll
        for (int q = 0; q < XP; ++q) *reinterpret_cast<f32x4 *>(buf + TN::LDS_ELEMS + xlds[q]) = r[q];
    };
    // this thread's share of the noise tile: coefficient row t / 16, features (t % 16) * 4 .. + 3 of the stage (8 bytes);
    // values for features past in_f meet zero columns of x
    const int nrow = t >> 4, nk = (t & 15) * 4;
    const int nlds = nrow * TN::LD + (((nk >> 3) ^ TN::swz(nrow)) * 8) + (nk & 7);
    const uint32_t nfirst = sq5_first((uint32_t)nk, (uint32_t)(m0 + nrow), p.seed);   // noise(i, m): first(i, m), + PN1 per feature
    auto hash_noise = [&](bf16_t *buf, int stage) {
        const uint32_t f0 = nfirst + (uint32_t)(stage * F_BK) * PN1;
        uint2 v;
        v.x = f32x2_to_bf16x2((float)(int32_t)sq5_tail(f0), (float)(int32_t)sq5_tail(f0 + PN1));
        v.y = f32x2_to_bf16x2((float)(int32_t)sq5_tail(f0 + 2u * PN1), (float)(int32_t)sq5_tail(f0 + 3u * PN1));
        *reinterpret_cast<uint2 *>(buf + nlds) = v;
    };
    f32x16 acc = zero16();
    f32x4 rx[2][XP];
    {
        f32x4 rx0[XP];
        load_x(rx0, 0);
        load_x(rx[1], 1);
        load_x(rx[0], 2);
        hash_noise(lds, 0);
        store_x(lds, rx0);
    }
    RDB_STAMP(1);
    auto stage_body = [&](int s, int u, bool more) {   // stage s in LDS buffer u (= s % 2); slot (u ^ 1) of rx holds stage s + 1
        bf16_t *cur = lds + u * STAGE, *oth = lds + (u ^ 1) * STAGE;
        __syncthreads();   // stage s is complete in `cur`; everybody has finished reading `oth` (stage s - 1)
        bf16x8 fa[4], fb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            fa[ks] = TN::frag(cur, 0, ks, lane);
            fb[ks] = TX::frag(cur + TN::LDS_ELEMS, wave * 32, ks, lane);
        }
        if (more) {
            store_x(oth, rx[u ^ 1]);
            load_x(rx[u ^ 1], s + 3);
            hash_noise(oth, s + 1);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks], fb[ks], acc, 0, 0, 0);
    };
    int s = 0;
    for (; s + 2 < nstage; s += 2) {
        stage_body(s, 0, true);
        stage_body(s + 1, 1, true);
    }
    stage_body(s, 0, s + 1 < nstage);
    if (s + 1 < nstage) stage_body(s + 1, 1, false);
    finish_units();
    __syncthreads();   // the last stage's fragment reads are done: the tile buffers may be reused
    RDB_STAMP(2);
    // The tile D[a = coefficient][b = token] goes to LDS once, as bf16 rows of tokens (LD elements apart), and leaves in
    // up to two orders.  Rows of tokens past the end and coefficients past k hold zeros or finite values: every byte of the
    // state's z pieces is written, so that their consumers may multiply padding with zeros.
    constexpr int LD = KZ_BM + 8;
    {
        const int r = lane & 31, g = lane >> 5, b = wave * 32 + r;
#pragma unroll
        for (int jq = 0; jq < 4; ++jq)
            store4<bf16_t>(lds + b * LD + 8 * jq + 4 * g, acc[jq * 4 + 0] * INV_2_31, acc[jq * 4 + 1] * INV_2_31, acc[jq * 4 + 2] * INV_2_31,
                           acc[jq * 4 + 3] * INV_2_31);
    }
    __syncthreads();
    constexpr int PIECES = KZ_BM * KZ_BT / 8;
    {
        // rows = tokens, k = coefficients: a piece is 8 coefficients of one token, neighbouring lanes take neighbouring tokens
        // device scope (written through): blocks of this very launch on other dies may be waiting for the tile
        const int ksteps = p.kpad >> 4;
        const __amdgpu_buffer_rsrc_t rs_zf = __builtin_amdgcn_make_buffer_rsrc(p.zf, 0, (int)((int64_t)p.tok32 * p.kpad * 2), 0x00020000);
#pragma unroll
        for (int q = 0; q < PIECES / KZ_THREADS; ++q) {
            const int idx = q * KZ_THREADS + t, b = idx % KZ_BT, a = (idx / KZ_BT) * 8;
            const int gb = tok0 + b, ga = m0 + a;
            if (gb < p.tok32)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, *reinterpret_cast<const f32x4 *>(lds + b * LD + a)), rs_zf,
                                                       (int)((((gb >> 5) * ksteps + (ga >> 4)) * 512 + (((ga >> 3) & 1) * 32 + (gb & 31)) * 8) * 2), 0,
                                                       SCOPE_DEVICE);
        }
    }
    {
        // rows = coefficients, k = tokens: the LDS transpose read turns 16 token rows x 32 coefficients into the fragment
        const int tsteps = p.tok64 >> 4, sl = lane & 15, qq = (lane >> 4) & 1, g = lane >> 5;
#pragma unroll
        for (int q = 0; q < KZ_BT / 16 / (KZ_THREADS / 64); ++q) {
            const int ks = wave * (KZ_BT / 16 / (KZ_THREADS / 64)) + q;   // token k-step inside the tile
            if (tok0 + ks * 16 >= p.tok64) continue;
            const bf16_t *src = lds + (ks * 16 + g * 8 + (sl >> 2)) * LD + qq * 16 + (sl & 3) * 4;
            Frag8 f;
            f.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(src));
            f.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(src + 4 * LD));
            store_stream(reinterpret_cast<f32x4 *>(p.ztf + ((int64_t)(m0 >> 5) * tsteps + (tok0 >> 4) + ks) * 512 + lane * 8), f.f4);
        }
    }
    if (p.sync) {
        unsigned long long *slots = p.sync + (int64_t)(w / p.tiles_m) * (p.tiles_m + 1);
        if (w % p.tiles_m == 0 && t == 0)
            __hip_atomic_store(reinterpret_cast<unsigned int *>(slots + p.tiles_m), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        publish_tag(slots + (w % p.tiles_m), p.sync_tag);
    }
    RDB_STAMP(3);
}

__global__ __launch_bounds__(KZ_THREADS, 1) void factored_z_kernel(ZParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    z_block(p, smem_raw, blockIdx.x, gridDim.x);
}

// ----------------------------------------------------------------------------------------------- y = z . C^T
// Any k (the kernel for k > 256).  tile: 128 output features (rows "a", C staged through LDS) x 128 tokens (rows "b", z taken
// from its fragment-ordered copy straight into registers), contraction over k; two blocks per CU.
constexpr int KY_BO = 128, KY_BT = 128;

struct YParams {
    const bf16_t *z;   // fragment order, rows = tokens (padded to tok32), k padded to kpad
    const bf16_t *coef;
    const bf16_t *bias;
    bf16_t *y;
    int64_t ldy;
    int tokens, out_f, k, kpad, tok32;
    int tiles_o, tiles_t;
};

__global__ __launch_bounds__(256, 2) void factored_y_kernel(YParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, output tile), output tile fastest: neighbours share the z tile, a die shares C
    const int w = xcd_work_item(blockIdx.x, p.tiles_o * p.tiles_t);
    if (w >= p.tiles_o * p.tiles_t) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, wm = wave >> 1, wn = wave & 1;
    const int o0 = (w % p.tiles_o) * KY_BO, tok0 = (w / p.tiles_o) * KY_BT;
    f32x16 acc[KY_BO / 64][KY_BT / 64];
#pragma unroll
    for (int mi = 0; mi < KY_BO / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < KY_BT / 64; ++ni) acc[mi][ni] = zero16();
    GlobalOperand<KY_BO, F_BK, K_CONT> opc = {p.coef, (int64_t)p.k, o0, p.out_f, p.k, (int64_t)p.out_f * p.k};
    FragSource fz;   // this wave's 64 tokens; row blocks past tok32 fail the bounds check and read as zeros
    fz.init(p.z, (int64_t)p.tok32 * p.kpad, p.kpad >> 4, (tok0 + wn * 64) >> 5, lane);
    direct_mainloop<KY_BO / 64, KY_BT / 64, F_BK / 16, true, 2, 2, 2>(acc, lds, opc, fz, 0, (p.k + F_BK - 1) / F_BK, wm * 64, lane);
    store_tile_bf16<KY_BO, KY_BT>(acc, lds, p.y, p.ldy, o0, p.out_f, tok0, p.tokens, 1.0f, p.bias);
}

// ----------------------------------------------------------------------------------------------- y = z . C^T, k <= 256
// body in rdb_stationary.hpp: the projection of a token stays in registers (read in fragment order, as factored_z_kernel
// leaves it), the rows of C stream through LDS
template <int KG, bool BIAS> __global__ __launch_bounds__(ST_THREADS, 1) void factored_ys_kernel(StParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    stationary_block<KG, BIAS, false, true>(p, smem_raw, blockIdx.x);
}

// Projection and forward product in one launch: blocks 0 .. z_blocks - 1 project (z_block), the others multiply
// (stationary_block) and wait, tile by tile, for the tags of the projection blocks that feed them.  A multiplying block
// starts on a compute unit the moment a projecting block leaves it: no drain of the whole chip, no second launch in between.
struct ZYParams {
    ZParams z;
    StParams y;
    int z_blocks;   // a multiple of 8, so that both kinds keep their numbering over the dies
};

template <int KG, bool BIAS> __global__ __launch_bounds__(ST_THREADS, 1) void factored_zy_kernel(ZYParams p)
{
    static_assert(KZ_THREADS == ST_THREADS && KZ_BT == ST_BT, "one block size and one token tile for both kinds of block");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    if ((int)blockIdx.x < p.z_blocks)
        z_block(p.z, smem_raw, blockIdx.x, p.z_blocks);
    else
        stationary_block<KG, BIAS, false, true>(p.y, smem_raw, blockIdx.x - p.z_blocks);
}

// ----------------------------------------------------------------------------------------------- dC = dy^T . z
// body in rdb_blocks.hpp (dc_block_direct)
__global__ __launch_bounds__(256, 1) void factored_dc_kernel(DcParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    dc_block_direct(p, reinterpret_cast<bf16_t *>(smem_raw), blockIdx.x);
}

// ----------------------------------------------------------------------------------------------- host side
// What every factored kernel needs of the layer; coef_dtype is checked by the callers that read coefficients.
static bool factored_shape_ok(const rdb_linear_desc *d) { return proj_layout(d).ok; }
// AUTO takes the factored form up to 16 times the flops of one product on a stored W (k (in + out) < 16 in out).  Its flops break
// even with that product at k = in out / (in + out), but what AUTO would run instead is a kernel that forms W on chip, and
// measured against those the two factored products stay ahead far beyond that point (2048 tokens, 1024 -> 1024, k = 1024:
// forward 23 us against 164 us, coefficient gradient 36 us against 157 us; k = 1024 on 256 -> 256: 19 against 38, 22 against 72).
static bool cheaper_factored(const rdb_linear_desc *d) { return d->k * (d->in_f + d->out_f) < 16 * d->in_f * d->out_f; }
static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

int64_t linear_projection_bytes(const rdb_linear_desc *d) { return proj_layout(d).bytes; }

static bf16_t *state_piece(const void *state, int64_t off) { return reinterpret_cast<bf16_t *>(static_cast<char *>(const_cast<void *>(state)) + off); }

// Fills the coefficient-gradient parameters that name the projection state's pieces.
void dc_params_from_state(DcParams &p, const void *state, const rdb_linear_desc *d)
{
    const ProjLayout L = proj_layout(d);
    p.ztf = state_piece(state, L.ztf_off);
    p.tsteps = (int)(L.tok64 / 16);
    p.kpad = L.kpad;
}

// The entry points below return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
// state <- projection of x (z for the forward product, z transposed for the coefficient gradient) and, when coef is given,
// the transposed coefficients for the input gradient.
int linear_fwd_projected(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                         hipStream_t s);

static bool fill_z_params(ZParams &p, void *state, const void *x, int64_t ldx, const void *coef, const rdb_linear_desc *d)
{
    const ProjLayout L = proj_layout(d);
    if (!L.ok || d->tokens * ldx >= (1ll << 29) || ldx % 8 || !aligned16(x) || !aligned16(state)) return false;
    if (coef && d->coef_dtype != RDB_BF16) coef = nullptr;   // the transposed copy is an operand of the bf16 kernels only
    p.x = (const bf16_t *)x;
    p.coef = (const bf16_t *)coef;
    p.zf = state_piece(state, L.zf_off);
    p.ztf = state_piece(state, L.ztf_off);
    p.ctf = state_piece(state, L.ctf_off);
    p.flag = reinterpret_cast<uint32_t *>(state);
    p.ldx = ldx;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.kpad = L.kpad;
    p.tok32 = (int)L.tok32;
    p.tok64 = (int)L.tok64;
    p.out64 = (int)L.out64;
    p.seed = d->seed;
    p.tiles_m = L.kpad / KZ_BM;   // every coefficient row block of the padded pieces is written
    p.tiles_t = (int)cdiv(d->tokens, KZ_BT);
    p.sync = nullptr;
    p.sync_tag = 0;
    return true;
}

static size_t z_smem() { return engine_smem<KZ_BM, KZ_BT, F_BK, K_CONT, K_CONT>(); }

int linear_project(void *state, const void *x, int64_t ldx, const void *coef, const rdb_linear_desc *d, hipStream_t s)
{
    ZParams p;
    if (!fill_z_params(p, state, x, ldx, coef, d)) return RDB_E_UNSUPPORTED;
    const size_t smem = z_smem();
    if (int rl = reserve_lds(reinterpret_cast<const void *>(factored_z_kernel), smem, "factored_z_kernel")) return rl;
    factored_z_kernel<<<xcd_grid_size(p.tiles_m * p.tiles_t), KZ_THREADS, smem, s>>>(p);
    return check_launch("factored_z_kernel");
}

// The forward product's parameters when the contraction of a token fits in registers (z in fragment order); returns the
// number of work items, 0 when the request does not fit.
static int fill_ys_params(StParams &q, void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d,
                          int num_cus)
{
    const ProjLayout L = proj_layout(d);
    if (!L.ok || !L.fits_regs || d->coef_dtype != RDB_BF16 || ldy % 8 || !aligned16(y) || !aligned16(state) || !aligned16(coef)) return 0;
    if (((uintptr_t)bias & 7) || d->tokens * ldy >= (1ll << 29)) return 0;
    q.z = state_piece(state, L.zf_off);
    q.coef = (const bf16_t *)coef;
    q.bias = (const bf16_t *)bias;
    q.y = (bf16_t *)y;
    q.ldy = ldy;
    q.k = (int)d->k;
    q.seed = 0;
    return make_stationary_grid(q, d->tokens, d->out_f, num_cus);
}

template <int KG, bool BIAS> static int launch_zy(const ZYParams &p, int y_items, hipStream_t s)
{
    const size_t smem = std::max(z_smem(), stationary_smem(KG));
    if (int rl = reserve_lds(reinterpret_cast<const void *>(factored_zy_kernel<KG, BIAS>), smem, "factored_zy_kernel")) return rl;
    factored_zy_kernel<KG, BIAS><<<p.z_blocks + xcd_grid_size(y_items), ST_THREADS, smem, s>>>(p);
    return check_launch("factored_zy_kernel");
}

// state <- projection of x (with the transposed coefficients if with_ct), y <- forward product, in one launch when the
// contraction of a token fits in registers (k <= 256), otherwise in two.
int linear_project_fwd(void *y, int64_t ldy, void *state, const void *x, int64_t ldx, const void *coef, bool with_ct, const void *bias,
                       const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    ZYParams p;
    if (!fill_z_params(p.z, state, x, ldx, with_ct ? coef : nullptr, d)) return RDB_E_UNSUPPORTED;
    const int y_items = fill_ys_params(p.y, y, ldy, state, coef, bias, d, num_cus);
    if (!y_items || p.z.tiles_m > 64 || !one_launch_mode()) {
        // check the second call's conditions before the first launch, so that a refusal leaves nothing half done
        if (d->coef_dtype != RDB_BF16 || ldy % 8 || !aligned16(y) || !aligned16(coef)) return RDB_E_UNSUPPORTED;
        if (((uintptr_t)bias & 7) || d->tokens * ldy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
        if (int rc = linear_project(state, x, ldx, with_ct ? coef : nullptr, d, s)) return rc;
        return linear_fwd_projected(y, ldy, state, coef, bias, d, num_cus, s);
    }
    const ProjLayout L = proj_layout(d);
    p.z.sync = reinterpret_cast<unsigned long long *>(static_cast<char *>(state) + L.sync_off);
    p.z.sync_tag = next_sync_tag();
    p.y.sync = p.z.sync;
    p.y.sync_tag = p.z.sync_tag;
    p.y.sync_n = p.z.tiles_m;
    p.y.sync_wait.err = reinterpret_cast<unsigned int *>(state) + 1;
    p.y.sync_wait.polls = SYNC_SPIN_LIMIT;
    if (int rc = sync_giveups_ptr(&p.y.sync_wait.giveups)) return rc;
    p.z_blocks = xcd_grid_size(p.z.tiles_m * p.z.tiles_t);
    const int kg = (int)cdiv(d->k, 64);
    if (bias) {
        switch (kg) {
        case 1: return launch_zy<1, true>(p, y_items, s);
        case 2: return launch_zy<2, true>(p, y_items, s);
        case 3: return launch_zy<3, true>(p, y_items, s);
        default: return launch_zy<4, true>(p, y_items, s);
        }
    }
    switch (kg) {
    case 1: return launch_zy<1, false>(p, y_items, s);
    case 2: return launch_zy<2, false>(p, y_items, s);
    case 3: return launch_zy<3, false>(p, y_items, s);
    default: return launch_zy<4, false>(p, y_items, s);
    }
}

// Test hook: only the multiplying blocks of the one-launch forward, waiting (at most `polls` polls each) for a tag that
// nobody publishes on `state`.  Every block gives up, fills its share of y with NaN and reports to the give-up counter.
int selftest_giveup_factored(void *y, int64_t ldy, void *state, const void *coef, const rdb_linear_desc *d, int num_cus, int polls, hipStream_t s)
{
    StParams q;
    const int items = fill_ys_params(q, y, ldy, state, coef, nullptr, d, num_cus);
    const ProjLayout L = proj_layout(d);
    if (!items || L.kpad / KZ_BM > 64) return RDB_E_UNSUPPORTED;
    q.sync = reinterpret_cast<unsigned long long *>(static_cast<char *>(state) + L.sync_off);
    q.sync_tag = next_sync_tag();
    q.sync_n = L.kpad / KZ_BM;
    q.sync_wait.err = reinterpret_cast<unsigned int *>(state) + 1;
    q.sync_wait.polls = polls;
    if (int rc = sync_giveups_ptr(&q.sync_wait.giveups)) return rc;
    const int kg = (int)cdiv(d->k, 64);
    const size_t smem = stationary_smem(kg);
    switch (kg) {
    case 1: return launch_stationary(factored_ys_kernel<1, false>, q, items, smem, s, "factored_ys_kernel<1> (self-test)");
    case 2: return launch_stationary(factored_ys_kernel<2, false>, q, items, smem, s, "factored_ys_kernel<2> (self-test)");
    case 3: return launch_stationary(factored_ys_kernel<3, false>, q, items, smem, s, "factored_ys_kernel<3> (self-test)");
    default: return launch_stationary(factored_ys_kernel<4, false>, q, items, smem, s, "factored_ys_kernel<4> (self-test)");
    }
}

int linear_fwd_projected(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                         hipStream_t s)
{
    const ProjLayout L = proj_layout(d);
    if (!L.ok || d->coef_dtype != RDB_BF16 || ldy % 8 || !aligned16(y) || !aligned16(state) || !aligned16(coef)) return RDB_E_UNSUPPORTED;
    const bf16_t *zf = state_piece(state, L.zf_off);
    if (L.fits_regs) {   // the contraction of a token fits in registers
        StParams q;
        const int items = fill_ys_params(q, y, ldy, state, coef, bias, d, num_cus);
        if (!items) return RDB_E_UNSUPPORTED;
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
    if (big_fwd_applies(d, num_cus)) return linear_fwd_big(y, ldy, state, coef, bias, d, num_cus, s);
    YParams p;
    p.z = zf;
    p.coef = (const bf16_t *)coef;
    p.bias = (const bf16_t *)bias;
    p.y = (bf16_t *)y;
    p.ldy = ldy;
    p.tokens = (int)d->tokens;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.kpad = L.kpad;
    p.tok32 = (int)L.tok32;
    p.tiles_o = (int)cdiv(d->out_f, KY_BO);
    p.tiles_t = (int)cdiv(d->tokens, KY_BT);
    return launch_engine(factored_y_kernel, p, p.tiles_o * p.tiles_t, engine_smem<KY_BO, KY_BT, F_BK, K_CONT, K_CONT>(), s, "factored_y_kernel");
}

// dcoef must have been zeroed on the same stream.
int linear_dcoef_projected(float *dcoef, const void *dy, int64_t lddy, const void *state, const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    if (!factored_shape_ok(d) || d->tokens * lddy >= (1ll << 29) || lddy % 8 || !aligned16(dy) || !aligned16(state)) return RDB_E_UNSUPPORTED;
    DcParams p;
    const int items = make_dc_params(p, dcoef, dy, lddy, d, num_cus);
    dc_params_from_state(p, state, d);
    return launch_engine(factored_dc_kernel, p, items, engine_smem<KD_BO, KD_BM, F_BK, M_CONT, M_CONT>(), s,
                         "factored_dc_kernel");
}

// y = (x . N^T) . C^T with the projection state in the workspace.
int linear_fwd_factored(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                        const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (scale_bias || d->coef_dtype != RDB_BF16 || !factored_shape_ok(d)) return RDB_E_UNSUPPORTED;  // the random-bias term is not low rank
    if (!workspace || workspace_bytes < linear_projection_bytes(d)) return RDB_E_UNSUPPORTED;
    if (d->algo == RDB_ALGO_AUTO && !cheaper_factored(d)) return RDB_E_UNSUPPORTED;
    // check everything before the first launch, so that a refusal leaves nothing half done
    if (d->tokens * ldx >= (1ll << 29) || ldx % 8 || ldy % 8 || !aligned16(x) || !aligned16(coef) || !aligned16(y) || !aligned16(workspace))
        return RDB_E_UNSUPPORTED;
    if (((uintptr_t)bias & 7) || d->tokens * ldy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    return linear_project_fwd(y, ldy, workspace, x, ldx, coef, false, bias, d, num_cus, s);
}

// dC = dy^T . (x . N^T) with the projection state in the workspace; dcoef must have been zeroed on the same stream.
int linear_dcoef_factored(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus,
                          void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!factored_shape_ok(d)) return RDB_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < linear_projection_bytes(d)) return RDB_E_UNSUPPORTED;
    if (d->algo == RDB_ALGO_AUTO && !cheaper_factored(d)) return RDB_E_UNSUPPORTED;
    if (d->tokens * ldx >= (1ll << 29) || d->tokens * lddy >= (1ll << 29) || ldx % 8 || lddy % 8 || !aligned16(x) || !aligned16(dy) ||
        !aligned16(workspace))
        return RDB_E_UNSUPPORTED;
    int rc = linear_project(workspace, x, ldx, nullptr, d, s);
    if (rc) return rc;
    return linear_dcoef_projected(dcoef, dy, lddy, workspace, d, num_cus, s);
}

}  // namespace rdb
