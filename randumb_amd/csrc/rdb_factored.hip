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
// When k is at most 256 the whole contraction of a token fits in registers: a wave keeps the MFMA fragments of its 32 tokens
// of z (read once) and the block walks over the output features in units of 64 rows of C.  Per unit only the C tile goes
// through LDS (prefetched in registers, two LDS buffers, one barrier).  The epilogue of a unit (bias, rounding to bf16,
// transposition through a wave-private LDS patch, 128-byte row stores) is issued between the MFMAs of the next unit, from
// a second set of accumulators, and a block has eight waves, two to a SIMD, so that one wave's waits and vector work run
// under the other's matrix work.  One block per CU; the grid is (token tiles of 256) x (splits of the output range).
constexpr int YS_BT = 256, YS_BO = 64, YS_STG_LD = YS_BO + 8, YS_WAVES = 8, YS_THREADS = YS_WAVES * 64, YS_TW = YS_BT / YS_WAVES;

struct YSParams {
    const bf16_t *z;
    const bf16_t *coef;
    const bf16_t *bias;
    bf16_t *y;
    int64_t ldy;
    int tokens, out_f, k;
    int tiles_t, splits, units_per_split;
};

template <int KG, bool BIAS> struct YSBlock {
    static constexpr int kpad = KG * 64, ldk = kpad + 8, cpr = kpad / 8, ncp = YS_BO * cpr, NQ = ncp / YS_THREADS;
    const YSParams &p;
    bf16_t *Cs;   // [2][64 o][ldk]
    bf16_t *stg;  // this wave's [32 tok][72]
    int lane, r, g, unit0, nunits;
    __amdgpu_buffer_rsrc_t rs_c, rs_y, rs_b;
    f32x4 rc[NQ];
    int t;
    bf16x8 zf[KG * 4];
    uint2 braw[2][4];   // bias of the unit whose epilogue comes next: four output features per (mi, jq) of this lane
    int tok_y;          // token of the row piece this lane stores in step 0 of the epilogue; step q: 8 q further
    uint32_t off_y;     // its byte offset in y at output feature 0

    __device__ __forceinline__ void issue(int unit)
    {   // global -> registers for a C tile; rows past out_f read as zeros
        const int o0 = unit * YS_BO, left = p.out_f - o0;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int idx = q * YS_THREADS + t, co = idx / cpr, cm = (idx % cpr) * 8;   // cpr is a compile-time constant
            const uint32_t a = (co < left && cm < p.k) ? (uint32_t)(((o0 + co) * p.k + cm) * 2) : BUFFER_OOB;
            rc[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_c, (int)a, 0, 0));
        }
    }

    // One step of the pipeline: the MFMAs of unit u into `cur` (MMA) and, between them, the epilogue of unit u - 1 from `prev` (EPI).
    template <bool MMA, bool EPI> __device__ __forceinline__ void step(f32x16 (&cur)[2], const f32x16 (&prev)[2], int u)
    {
        bf16_t *cs = Cs + (u & 1) * YS_BO * ldk;
        if (MMA) {
            __syncthreads();   // the C tile of this unit is in `cs` (written at the end of the step before), the other buffer is free
            if (u + 1 < nunits) issue(unit0 + u + 1);
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) cur[mi] = zero16();
        }
        const int o0 = (unit0 + u - 1) * YS_BO;  // of the unit in `prev`
        // The bias of unit u is fetched now and used by the next step.  Vector memory operations retire in order, so a wait
        // for a load also waits for every store issued before it: all loads of a step are issued before its stores, the C
        // tile is taken out of its registers at the end of the step (a wait that lets the step's stores stay in flight) and
        // the bias in the next step, when those stores have had a whole unit's time to drain.
        uint2 bnow[2][4];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                bnow[mi][jq] = braw[mi][jq];
                if (MMA && BIAS) {   // out_f is a multiple of 8 and the feature index of 4: the four values exist together or not at all
                    const int o = o0 + YS_BO + mi * 32 + 8 * jq + 4 * g;
                    braw[mi][jq] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(rs_b, o < p.out_f ? o * 2 : (int)BUFFER_OOB, 0, 0));
                }
            }
        // the epilogue in 10 small operations, so that few values are in flight at a time: 8 x (accumulators of 8 output features
        // -> + bias -> bf16 -> patch[tok][o]), then 2 x (16 tokens: rows of 128 bytes out of the patch)
        auto epilogue_op = [&](int op) {
            if (op < 8) {
                const int mi = op >> 2, jq = op & 3;
                const uint2 b = bnow[mi][jq];
                const float b0 = __uint_as_float(b.x << 16), b1 = __uint_as_float(b.x & 0xffff0000u);
                const float b2 = __uint_as_float(b.y << 16), b3 = __uint_as_float(b.y & 0xffff0000u);
                bf16_t *dst = stg + r * YS_STG_LD + mi * 32 + 8 * jq + 4 * g;
                const f32x16 &a = prev[mi];
                if (BIAS)
                    store4<bf16_t>(dst, a[jq * 4 + 0] + b0, a[jq * 4 + 1] + b1, a[jq * 4 + 2] + b2, a[jq * 4 + 3] + b3);
                else
                    store4<bf16_t>(dst, a[jq * 4 + 0], a[jq * 4 + 1], a[jq * 4 + 2], a[jq * 4 + 3]);
                if (op == 7) __builtin_amdgcn_wave_barrier();  // LDS serves a wave's instructions in order: the reads see these writes
            } else {
                const int h = op - 8;
                f32x4 v[2];
#pragma unroll
                for (int q = 0; q < 2; ++q) v[q] = *reinterpret_cast<const f32x4 *>(stg + ((h * 2 + q) * 8 + (lane >> 3)) * YS_STG_LD + (lane & 7) * 8);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int qq = h * 2 + q;
                    const uint32_t a = (o0 + (lane & 7) * 8 < p.out_f && tok_y + qq * 8 < p.tokens)
                                           ? off_y + (uint32_t)(qq * 8 * (int)p.ldy * 2 + o0 * 2) : BUFFER_OOB;
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v[q]), rs_y, (int)a, 0, 0);
                }
                if (op == 9) __builtin_amdgcn_wave_barrier();
            }
        };
        const bf16_t *pa = cs + r * ldk + g * 8;
        constexpr int GK = 2, NG = KG * 4 / GK;   // groups of GK k-steps (2 GK MFMAs); the fragments of the next group are read meanwhile
        bf16x8 fa[2][GK][2];
        auto rd = [&](int grp) {
#pragma unroll
            for (int ks = 0; ks < GK; ++ks)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
                    fa[grp & 1][ks][mi] = *reinterpret_cast<const bf16x8 *>(pa + mi * 32 * ldk + (grp * GK + ks) * 16);
        };
        if (MMA) rd(0);
#pragma unroll
        for (int grp = 0; grp < NG; ++grp) {
            if (MMA && grp + 1 < NG) rd(grp + 1);
            __builtin_amdgcn_sched_barrier(0);
            if (MMA) {
#pragma unroll
                for (int ks = 0; ks < GK; ++ks)
#pragma unroll
                    for (int mi = 0; mi < 2; ++mi)
                        cur[mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[grp & 1][ks][mi], zf[grp * GK + ks], cur[mi], 0, 0, 0);
            }
            if (EPI) {
#pragma unroll
                for (int op = 0; op < 10; ++op)
                    if (op * NG / 10 == grp) epilogue_op(op);
            }
            if (MMA && EPI) {   // one MFMA, then a share of the epilogue's vector, LDS and store instructions
#pragma unroll
                for (int i = 0; i < 2 * GK; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002 | 0x080 | 0x040, 30 / (NG * GK) + 3, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MMA && u + 1 < nunits) {
            bf16_t *cn = Cs + ((u + 1) & 1) * YS_BO * ldk;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const int idx = q * YS_THREADS + t;
                *reinterpret_cast<f32x4 *>(cn + (idx / cpr) * ldk + (idx % cpr) * 8) = rc[q];
            }
        }
    }
};

template <int KG, bool BIAS> __global__ __launch_bounds__(YS_THREADS, 1) void factored_ys_kernel(YSParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    typedef YSBlock<KG, BIAS> B;
    const int t = threadIdx.x, wave = t >> 6;
    // work item = (token tile, split), split fastest: neighbours share the z tile, everyone shares C
    const int w = xcd_work_item(blockIdx.x, p.tiles_t * p.splits);
    if (w >= p.tiles_t * p.splits) return;
    B b = {p};
    b.Cs = reinterpret_cast<bf16_t *>(smem_raw);
    b.stg = b.Cs + 2 * YS_BO * B::ldk + wave * YS_TW * YS_STG_LD;
    b.lane = t & 63;
    b.r = b.lane & 31;
    b.g = b.lane >> 5;
    const int tok0 = (w / p.splits) * YS_BT + wave * YS_TW;  // first token of this wave
    b.unit0 = (w % p.splits) * p.units_per_split;
    b.nunits = min(p.units_per_split, (p.out_f + YS_BO - 1) / YS_BO - b.unit0);
    if (b.nunits <= 0) return;
    b.rs_c = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.coef), 0, (int)((int64_t)p.out_f * p.k * 2), 0x00020000);
    b.rs_y = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, (int)(((int64_t)(p.tokens - 1) * p.ldy + p.out_f) * 2), 0x00020000);
    b.rs_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.bias), 0, p.bias ? p.out_f * 2 : 0, 0x00020000);  // no bias: zeros
    const __amdgpu_buffer_rsrc_t rs_z =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.z), 0, (int)((int64_t)p.tokens * p.k * 2), 0x00020000);
    b.t = t;
    b.issue(b.unit0);
    // z fragments: operand "b" (rows = tokens); tokens past the end and coefficients past k read as zeros.  A lane's fragment
    // pieces lie 16 bytes here, 16 bytes there; read straight from global memory that costs a cache line per lane and
    // instruction, so the tile goes through LDS (the C buffers, not yet in use): whole rows in, fragments out, 128 tokens at a time.
    {
        constexpr int ZQ = 128 * B::cpr / YS_THREADS;
        bf16_t *zs = b.Cs;
        const int btok0 = (w / p.splits) * YS_BT;
        f32x4 zr[2][ZQ];   // both halves are requested at once: one trip to memory
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int q = 0; q < ZQ; ++q) {
                const int idx = q * YS_THREADS + t, row = idx / B::cpr, cm = (idx % B::cpr) * 8, tok = btok0 + h * 128 + row;
                const uint32_t a = (tok < p.tokens && cm < p.k) ? (uint32_t)(((int64_t)tok * p.k + cm) * 2) : BUFFER_OOB;
                zr[h][q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_z, (int)a, 0, 0));
            }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int q = 0; q < ZQ; ++q) {
                const int idx = q * YS_THREADS + t;
                *reinterpret_cast<f32x4 *>(zs + (idx / B::cpr) * B::ldk + (idx % B::cpr) * 8) = zr[h][q];
            }
            __syncthreads();
            if ((wave >> 2) == h) {
#pragma unroll
                for (int ks = 0; ks < KG * 4; ++ks)
                    b.zf[ks] = *reinterpret_cast<const bf16x8 *>(zs + ((wave & 3) * YS_TW + b.r) * B::ldk + ks * 16 + b.g * 8);
            }
            __syncthreads();
        }
#pragma unroll
        for (int q = 0; q < B::NQ; ++q) {   // first C tile; the barrier at the top of step 0 publishes it
            const int idx = q * YS_THREADS + t;
            *reinterpret_cast<f32x4 *>(zs + (idx / B::cpr) * B::ldk + (idx % B::cpr) * 8) = b.rc[q];
        }
    }
    b.tok_y = tok0 + (b.lane >> 3);
    b.off_y = (uint32_t)(((int64_t)b.tok_y * p.ldy + (b.lane & 7) * 8) * 2);  // only used when the token exists: below 2^30

    // step s: MFMAs of unit s (while there is one) and the epilogue of unit s - 1; even steps accumulate in A, odd ones in B
    f32x16 accA[2], accB[2];
    const int n = b.nunits;
    b.template step<true, false>(accA, accB, 0);
    int s = 1;
    for (; s + 1 < n; s += 2) {
        b.template step<true, true>(accB, accA, s);
        b.template step<true, true>(accA, accB, s + 1);
    }
    if (s < n) {   // s == n - 1, odd
        b.template step<true, true>(accB, accA, s);
        b.template step<false, true>(accA, accB, s + 1);
    } else {       // s == n, odd
        b.template step<false, true>(accB, accA, s);
    }
}

template <class K> static int launch_ys(K kernel, const YSParams &q, int items, size_t smem, hipStream_t s, const char *name)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return set_error((int)e, "%s: cannot reserve %zu bytes of LDS: %s", name, smem, hipGetErrorString(e));
    kernel<<<xcd_grid_size(items), YS_THREADS, smem, s>>>(q);
    return check_launch(name);
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
    if (d->k <= 256 && ((uintptr_t)bias & 7) == 0 && d->tokens * ldy < (1ll << 29)) {  // the contraction of a token fits in registers
        YSParams q;
        q.z = (const bf16_t *)z;
        q.coef = (const bf16_t *)coef;
        q.bias = (const bf16_t *)bias;
        q.y = (bf16_t *)y;
        q.ldy = ldy;
        q.tokens = (int)d->tokens;
        q.out_f = (int)d->out_f;
        q.k = (int)d->k;
        q.tiles_t = (int)cdiv(d->tokens, YS_BT);
        const int units = (int)cdiv(d->out_f, YS_BO);
        int splits = (int)cdiv(num_cus, q.tiles_t);   // about one block per CU
        if (splits > units) splits = units;
        q.units_per_split = (int)cdiv(units, splits);
        q.splits = (int)cdiv(units, q.units_per_split);
        const int kg = (int)cdiv(d->k, 64), items = q.tiles_t * q.splits;
        const size_t smem = ((size_t)2 * YS_BO * (kg * 64 + 8) + YS_BT * YS_STG_LD) * sizeof(bf16_t);
        if (bias) {
            switch (kg) {
            case 1: return launch_ys(factored_ys_kernel<1, true>, q, items, smem, s, "factored_ys_kernel<1,bias>");
            case 2: return launch_ys(factored_ys_kernel<2, true>, q, items, smem, s, "factored_ys_kernel<2,bias>");
            case 3: return launch_ys(factored_ys_kernel<3, true>, q, items, smem, s, "factored_ys_kernel<3,bias>");
            default: return launch_ys(factored_ys_kernel<4, true>, q, items, smem, s, "factored_ys_kernel<4,bias>");
            }
        }
        switch (kg) {
        case 1: return launch_ys(factored_ys_kernel<1, false>, q, items, smem, s, "factored_ys_kernel<1>");
        case 2: return launch_ys(factored_ys_kernel<2, false>, q, items, smem, s, "factored_ys_kernel<2>");
        case 3: return launch_ys(factored_ys_kernel<3, false>, q, items, smem, s, "factored_ys_kernel<3>");
        default: return launch_ys(factored_ys_kernel<4, false>, q, items, smem, s, "factored_ys_kernel<4>");
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
