// Products whose contraction index is the coefficient index, at most 256 long:
//
//   y[tok, o]  = sum_m z[tok, m] * C[o, m]                    (forward from the projection)
//   dx[tok, i] = sum_m t[tok, m] * noise(PRIME*i + m)         (second half of the input gradient, t = dy . C)
//
// The whole contraction of a token fits in registers: a wave keeps the MFMA fragments of its 32 tokens of the left operand
// (read once) and the block walks over the output features in units of 64.  Per unit only the right operand's tile, 64 rows
// of C or 64 hashed rows of noise, goes through LDS (two buffers, one barrier).  The epilogue of a unit (bias, rounding to
// bf16, transposition through a wave-private LDS patch, 128-byte row stores) is issued between the MFMAs of the next unit,
// from a second set of accumulators, and a block has eight waves, two to a SIMD, so that one wave's waits and vector work
// run under the other's matrix work.  One block per CU; the grid is (token tiles of 256) x (splits of the output range).
#pragma once
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

#ifndef RDB_Y_STORE_AUX
#define RDB_Y_STORE_AUX 2   // cache policy of the output row stores: non-temporal (y and dx are not read again by this library, and
                           // lines that do not linger in L2 need no write-back when the kernel ends: the next launch starts sooner)
#endif

constexpr int ST_BT = 256, ST_BO = 64, ST_STG_LD = ST_BO + 8, ST_WAVES = 8, ST_THREADS = ST_WAVES * 64, ST_TW = ST_BT / ST_WAVES;
constexpr int ST_KMAX = 256;

struct StParams {
    const bf16_t *z;     // left operand [tokens x k]: row-major, or (ZFRAG) in fragment order as store_tile_bf16_frag writes it,
                         // tokens padded to 32 and k to KG * 64, the noise flavour's 2^-31 already applied
    const bf16_t *coef;  // right operand [out_f x k] (not used when the right operand is noise)
    const bf16_t *bias;  // [out_f] or NULL
    bf16_t *y;           // [tokens x out_f], leading dimension ldy
    int64_t ldy;
    int tokens, out_f, k;
    int tiles_t, splits, units_per_split;
    uint32_t seed;       // noise flavour
    // ZFRAG only: NULL, or slots [token tile of 256][sync_n + 1] that earlier blocks of the same launch set to sync_tag when the
    // tile's share of z is in memory (the last slot of a tile counts the blocks that have seen them)
    unsigned long long *sync;
    unsigned long long sync_tag;
    int sync_n;
    SyncWait sync_wait;
};

// KG: k rounded up to groups of 64 (compile time: the k loop is one straight line of code).  NOISE: the right operand's
// rows are 2^31 * noise(PRIME*row + m), hashed into the tile; the producer of the left operand has scaled it by 2^-31
// (exact in bf16).
template <int KG, bool BIAS, bool NOISE> struct StBlock {
    static constexpr int kpad = KG * 64, ldk = kpad + 8, cpr = kpad / 8, ncp = ST_BO * cpr, NQ = ncp / ST_THREADS;
    const StParams &p;
    bf16_t *Cs;   // [2][64 rows][ldk]
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
        const int o0 = unit * ST_BO, left = p.out_f - o0;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int idx = q * ST_THREADS + t, co = idx / cpr, cm = (idx % cpr) * 8;   // cpr is a compile-time constant
            const uint32_t a = (co < left && cm < p.k) ? (uint32_t)(((o0 + co) * p.k + cm) * 2) : BUFFER_OOB;
            rc[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_c, (int)a, 0, 0));
        }
    }
    __device__ __forceinline__ void hash_piece(int unit, int q)
    {   // piece q of this thread in the noise tile of `unit`: 8 consecutive coefficients of one row; coefficients past k meet zeros
        const int idx = q * ST_THREADS + t, co = idx / cpr, cm = (idx % cpr) * 8;
        const uint32_t first = sq5_first((uint32_t)(unit * ST_BO + co), (uint32_t)cm, p.seed);
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * SQ5_N1);
        Frag8 f;
#pragma unroll
        for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
        rc[q] = f.f4;
    }
    __device__ __forceinline__ void hash_piece_all(int unit)
    {
#pragma unroll
        for (int q = 0; q < NQ; ++q) hash_piece(unit, q);
    }
    __device__ __forceinline__ void commit(bf16_t *cn)
    {   // registers -> LDS for the tile in rc
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int idx = q * ST_THREADS + t;
            *reinterpret_cast<f32x4 *>(cn + (idx / cpr) * ldk + (idx % cpr) * 8) = rc[q];
        }
    }

    // One step of the pipeline: the MFMAs of unit u into `cur` (MMA) and, between them, the epilogue of unit u - 1 from `prev` (EPI).
    template <bool MMA, bool EPI> __device__ __forceinline__ void step(f32x16 (&cur)[2], const f32x16 (&prev)[2], int u)
    {
        bf16_t *cs = Cs + (u & 1) * ST_BO * ldk;
        const bool more = u + 1 < nunits;
        if (MMA) {
            __syncthreads();   // the tile of this unit is in `cs` (written at the end of the step before), the other buffer is free
            if (!NOISE && more) issue(unit0 + u + 1);
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) cur[mi] = zero16();
        }
        const int o0 = (unit0 + u - 1) * ST_BO;  // of the unit in `prev`
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
                    const int o = o0 + ST_BO + mi * 32 + 8 * jq + 4 * g;
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
                bf16_t *dst = stg + r * ST_STG_LD + mi * 32 + 8 * jq + 4 * g;
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
                for (int q = 0; q < 2; ++q) v[q] = *reinterpret_cast<const f32x4 *>(stg + ((h * 2 + q) * 8 + (lane >> 3)) * ST_STG_LD + (lane & 7) * 8);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int qq = h * 2 + q;
                    const uint32_t a = (o0 + (lane & 7) * 8 < p.out_f && tok_y + qq * 8 < p.tokens)
                                           ? off_y + (uint32_t)(qq * 8 * (int)p.ldy * 2 + o0 * 2) : BUFFER_OOB;
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v[q]), rs_y, (int)a, 0, RDB_Y_STORE_AUX);
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
            if (NOISE && MMA && more) {   // the next unit's noise tile is hashed under this unit's MFMAs
#pragma unroll
                for (int q = 0; q < NQ; ++q)
                    if (q * NG / NQ == grp) hash_piece(unit0 + u + 1, q);
            }
            if (!NOISE && MMA && EPI) {   // one MFMA, then a share of the epilogue's vector, LDS and store instructions
#pragma unroll
                for (int i = 0; i < 2 * GK; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002 | 0x080 | 0x040, 30 / (NG * GK) + 3, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MMA && more) commit(Cs + ((u + 1) & 1) * ST_BO * ldk);
    }
};

// `block`: index of this block among the blocks that run this body; all ST_THREADS threads of the block must call.
template <int KG, bool BIAS, bool NOISE, bool ZFRAG = false>
__device__ __forceinline__ void stationary_block(const StParams &p, unsigned char *smem_raw, int block)
{
    typedef StBlock<KG, BIAS, NOISE> B;
    const int t = threadIdx.x, wave = t >> 6;
    // work item = (token tile, split), split fastest: neighbours share the left operand's tile, everyone shares the right operand
    const int w = xcd_work_item(block, p.tiles_t * p.splits);
    if (w >= p.tiles_t * p.splits) return;
    B b = {p};
    b.Cs = reinterpret_cast<bf16_t *>(smem_raw);
    b.stg = b.Cs + 2 * ST_BO * B::ldk + wave * ST_TW * ST_STG_LD;
    b.lane = t & 63;
    b.r = b.lane & 31;
    b.g = b.lane >> 5;
    const int tok0 = (w / p.splits) * ST_BT + wave * ST_TW;  // first token of this wave
    b.unit0 = (w % p.splits) * p.units_per_split;
    b.nunits = min(p.units_per_split, (p.out_f + ST_BO - 1) / ST_BO - b.unit0);
    if (b.nunits <= 0) return;
    RDB_STAMP(0);
    b.rs_c = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.coef), 0, NOISE ? 0 : (int)((int64_t)p.out_f * p.k * 2), 0x00020000);
    b.rs_y = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, (int)(((int64_t)(p.tokens - 1) * p.ldy + p.out_f) * 2), 0x00020000);
    b.rs_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.bias), 0, p.bias ? p.out_f * 2 : 0, 0x00020000);  // no bias: zeros
    b.t = t;
    if constexpr (ZFRAG) {
        // the fragments lie ready in memory, a k-step of a wave's 32 tokens in 1024 consecutive bytes: no staging, no barrier
        const int64_t padded = (int64_t)((p.tokens + 31) / 32) * 32 * B::kpad;
        const __amdgpu_buffer_rsrc_t rs_z = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.z), 0, (int)(padded * 2), 0x00020000);
        if (!NOISE) b.issue(b.unit0);
        if (p.sync) {   // z comes from earlier blocks of this launch
            // the verdict of the waiting wave reaches the others through a word of LDS that nothing else touches: the padding
            // at the end of the last row of the last wave's epilogue patch
            volatile int *verdict = reinterpret_cast<volatile int *>(b.Cs + 2 * ST_BO * B::ldk + ST_BT * ST_STG_LD) - 1;
            if (wave == 0) {
                unsigned long long *slots = p.sync + (int64_t)(w / p.splits) * (p.sync_n + 1);
                const bool there = await_tags(slots, p.sync_n, p.sync_tag, p.sync_wait);
                if (there) release_tags(slots, p.sync_n, reinterpret_cast<unsigned int *>(slots + p.sync_n), p.splits);
                if (b.lane == 0) *verdict = there ? 1 : 0;
            }
            __syncthreads();
            if (*verdict == 0) {
                // gave up: z of these tokens is not known to be in memory.  The block's share of y becomes NaN (a result
                // nobody can mistake for one) and the block leaves; the host learns of it from the give-up counter.
                const i32x4 nan8 = {0x7fc07fc0, 0x7fc07fc0, 0x7fc07fc0, 0x7fc07fc0};
                const int o_begin = b.unit0 * ST_BO, o_end = min(p.out_f, (b.unit0 + b.nunits) * ST_BO);
                const int pieces = (o_end - o_begin) / 8;   // out_f is a multiple of 8
                for (int e = t; e < ST_BT * pieces; e += ST_THREADS) {
                    const int tok = (w / p.splits) * ST_BT + e / pieces, o = o_begin + (e % pieces) * 8;
                    if (tok < p.tokens) __builtin_amdgcn_raw_buffer_store_b128(nan8, b.rs_y, (int)(((int64_t)tok * p.ldy + o) * 2), 0, 0);
                }
                return;
            }
        }
        const int tile = tok0 >> 5;
        if (p.sync) {   // written by other dies during this launch: read around this die's L2
#pragma unroll
            for (int ks = 0; ks < KG * 4; ++ks) {
                const uint32_t a = tok0 < p.tokens ? (uint32_t)(((tile * (KG * 4) + ks) * 512 + b.lane * 8) * 2) : BUFFER_OOB;
                b.zf[ks] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rs_z, (int)a, 0, SCOPE_DEVICE));
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < KG * 4; ++ks) {
                const uint32_t a = tok0 < p.tokens ? (uint32_t)(((tile * (KG * 4) + ks) * 512 + b.lane * 8) * 2) : BUFFER_OOB;
                b.zf[ks] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rs_z, (int)a, 0, 0));
            }
        }
        if (NOISE) b.hash_piece_all(b.unit0);   // the first noise tile is hashed while the loads are in flight
        b.commit(b.Cs);                          // first tile of the right operand; the barrier at the top of step 0 publishes it
    } else {
        static_assert(!NOISE, "the noise flavour takes its left operand in fragment order");
        const __amdgpu_buffer_rsrc_t rs_z =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.z), 0, (int)((int64_t)p.tokens * p.k * 2), 0x00020000);
        b.issue(b.unit0);
        // Left operand's fragments: operand "b" of the MFMA (rows = tokens); tokens past the end and coefficients past k read as
        // zeros.  A lane's fragment pieces lie 16 bytes here, 16 bytes there; read straight from global memory that costs a
        // cache line per lane and instruction, so a wave passes its 32 tokens through a patch of LDS of its own: whole rows in,
        // fragments out, half of the coefficients at a time, with no block-wide barrier.  The patches lie in the second tile
        // buffer and the epilogue patches, which nobody writes before the barrier of step 0.
        {
            constexpr int HK = B::kpad / 2, HLD = HK + 8, HQ = 32 * (HK / 8) / 64;   // half a row: HK coefficients; pieces per lane
            static_assert(ST_WAVES * 32 * HLD <= ST_BO * B::ldk + ST_BT * ST_STG_LD, "the waves' patches fit beside the first tile buffer");
            bf16_t *zs = b.Cs + ST_BO * B::ldk + wave * 32 * HLD;
            f32x4 zr[2][HQ];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < HQ; ++q) {
                    const int idx = q * 64 + b.lane, row = idx / (HK / 8), cm = h * HK + (idx % (HK / 8)) * 8, tok = tok0 + row;
                    const uint32_t a = (tok < p.tokens && cm < p.k) ? (uint32_t)(((int64_t)tok * p.k + cm) * 2) : BUFFER_OOB;
                    zr[h][q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_z, (int)a, 0, 0));
                }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int q = 0; q < HQ; ++q) {
                    const int idx = q * 64 + b.lane;
                    const f32x4 v = zr[h][q];
                    *reinterpret_cast<f32x4 *>(zs + (idx / (HK / 8)) * HLD + (idx % (HK / 8)) * 8) = v;
                }
                __builtin_amdgcn_wave_barrier();   // LDS serves a wave's instructions in order: the reads below see these writes
#pragma unroll
                for (int ks = 0; ks < KG * 2; ++ks)
                    b.zf[h * KG * 2 + ks] = *reinterpret_cast<const bf16x8 *>(zs + b.r * HLD + ks * 16 + b.g * 8);
                __builtin_amdgcn_wave_barrier();
            }
            b.commit(b.Cs);   // first tile of the right operand; the barrier at the top of step 0 publishes it
        }
    }
    b.tok_y = tok0 + (b.lane >> 3);
    b.off_y = (uint32_t)(((int64_t)b.tok_y * p.ldy + (b.lane & 7) * 8) * 2);  // only used when the token exists: below 2^30

    // step s: MFMAs of unit s (while there is one) and the epilogue of unit s - 1; even steps accumulate in A, odd ones in B
    f32x16 accA[2], accB[2];
    const int n = b.nunits;
    RDB_STAMP(1);
    b.template step<true, false>(accA, accB, 0);
    RDB_STAMP(2);
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
    RDB_STAMP(3);
}

// ----------------------------------------------------------------------------------------------- host side
inline size_t stationary_smem(int kg)
{
    return ((size_t)2 * ST_BO * (kg * 64 + 8) + ST_BT * ST_STG_LD) * sizeof(bf16_t);  // two tiles + the waves' patches
}

// Grid of the stationary kernels for [tokens x out_f]: about one block per compute unit.  Returns the number of work items.
inline int make_stationary_grid(StParams &q, int64_t tokens, int64_t out_f, int num_cus)
{
    q.tokens = (int)tokens;
    q.out_f = (int)out_f;
    q.sync = nullptr;   // the left operand comes from an earlier launch unless the caller says otherwise afterwards
    q.sync_tag = 0;
    q.sync_n = 0;
    q.sync_wait = {nullptr, nullptr, SYNC_SPIN_LIMIT};
    q.tiles_t = (int)cdiv(tokens, ST_BT);
    const int units = (int)cdiv(out_f, ST_BO);
    int splits = (int)cdiv(num_cus, q.tiles_t);
    if (splits > units) splits = units;
    q.units_per_split = (int)cdiv(units, splits);
    q.splits = (int)cdiv(units, q.units_per_split);
    return q.tiles_t * q.splits;
}

template <class K> inline int launch_stationary(K kernel, const StParams &q, int items, size_t smem, hipStream_t s, const char *name)
{
    if (int rl = reserve_lds(reinterpret_cast<const void *>(kernel), smem, name)) return rl;
    kernel<<<xcd_grid_size(items), ST_THREADS, smem, s>>>(q);
    return check_launch(name);
}

}  // namespace rdb
