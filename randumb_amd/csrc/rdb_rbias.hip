// The fused random bias beside the factored kernels.
//
// With scale_bias the weight is W = C . N + s . R,  R[o, i] = noise1d(o*in_f + i)  (src/rten_cpp/RandumbTensor.py:286-289;
// it is what the reference's default initialisation starts from: zero coefficients, random bias,
// src/rten_cpp/SillyLayers.py:122-133, 218-221).  R is a full-rank pseudorandom matrix, so its share of a product is a
// dense contraction whatever is done about C . N; the low-rank share keeps its factored kernels and this file adds
//     dx[t, i] += s * sum_o dy[t, o] * R[o, i]        (input gradient)
//     y[t, o]  += s * sum_i x[t, i]  * R[o, i]        (forward, where no kernel that forms W strips fits)
// on the tile engine with R as a hashed operand: a tile of 64 features x 256 tokens, R hashed once per block and
// stage straight into the pipeline's registers (as 2^31 * noise in bf16, the scale folded into the epilogue), two blocks
// per compute unit so that one block's hashing runs under the other's matrix work.  R never exists in memory.
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

int num_compute_units();   // of the current device (rdb_error.hip)

constexpr int RB_BI = 64, RB_BT = 256, RB_BK = 64;

// Hashed operand: element (row, k) = 2^31 * noise1d((row0 + row) * sR + k * sK) as bf16.
template <int ROWS, int BK> struct Noise1DOperand {
    typedef OperandTile<ROWS, BK, K_CONT> Tile;
    int row0;
    uint32_t sR, sK, seed;
    int k_begin;
    __device__ __forceinline__ void init(int kb) { k_begin = kb; }
    __device__ __forceinline__ void load_piece(f32x4 &reg, int p, int stage) const
    {
        const int idx = p * 256 + threadIdx.x, k0 = k_begin + stage * BK;
        const uint32_t row = (uint32_t)(row0 + idx / (BK / 8)), k = (uint32_t)(k0 + (idx % (BK / 8)) * 8);
        const uint32_t step = sK * SQ5_N1, first = (row * sR + k * sK) * SQ5_N1 + seed;
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * step);
        Frag8 f;
#pragma unroll
        for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
        reg = f.f4;
    }
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int stage) const
    {
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p) load_piece(regs[p], p, stage);
    }
};

// dst[t, a] += s * sum_c src[t, c] * noise1d(a * sR + c * sK):  the input gradient has a = input feature, c = output feature
// (sR = 1, sK = in_f), the forward a = output feature, c = input feature (sR = in_f, sK = 1).
struct RBiasParams {
    const bf16_t *dy;           // src [tokens x out_f (contraction)]
    const bf16_t *scale_bias;   // one bf16 value
    bf16_t *dx;                 // dst [tokens x in_f (columns)]
    int64_t lddy, lddx;
    int tokens, in_f, out_f;    // in_f: columns of dst, out_f: contraction length
    int tiles_i, tiles_t;
    uint32_t sR, sK;
    uint32_t seed;
    // DOT: the gradient of the scale on the side, d s = <src . R, other> = sum over the tile of the product (without s) times
    // other[tokens x in_f columns]; one partial sum per work item, in work-item order
    const bf16_t *other;
    int64_t ld_other;
    float *dot_part;
};

template <bool DOT> __global__ __launch_bounds__(256, 2) void rbias_add_kernel(RBiasParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    // work item = (token tile, feature tile), feature tile fastest: neighbours share the dy tile
    const int w = xcd_work_item(blockIdx.x, p.tiles_i * p.tiles_t);
    if (w >= p.tiles_i * p.tiles_t) return;
    const int i0 = (w % p.tiles_i) * RB_BI, tok0 = (w / p.tiles_i) * RB_BT;
    constexpr int MI = RB_BI / 32, NI = RB_BT / 128;
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = zero16();
    // "A": 2^31 * R, rows = columns of dst: the noise index moves by sR per row and by sK per contraction value
    Noise1DOperand<RB_BI, RB_BK> opr = {i0, p.sR, p.sK, p.seed};
    // "B": src[tok][c]; contraction values past the end read as zeros, whatever the hash says there
    GlobalOperand<RB_BT, RB_BK, K_CONT> opdy = {p.dy, p.lddy, tok0, p.tokens, p.out_f, (int64_t)(p.tokens - 1) * p.lddy + p.out_f};
    gemm_mainloop<RB_BI, RB_BT, RB_BK, 1, 2, 1>(acc, lds, opr, opdy, 0, (p.out_f + RB_BK - 1) / RB_BK);
    // dx += s * (2^-31 * acc), through LDS as fp32 so that every lane updates 8 consecutive features of a token's row
    // (2^-31 * acc is exact, so the product with s is rounded once, as s * 2^-31 times acc would be)
    const float sval = bf16_to_f32(*p.scale_bias);
    constexpr float scale = 4.656612873077392578125e-10f;
    constexpr int LDF = RB_BI + 4;   // floats per token row of the staging tile
    float *stage = reinterpret_cast<float *>(smem_raw);
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const int b = wave * NI * 32 + ni * 32 + r, a = mi * 32 + 8 * jq + 4 * g;
                const f32x4 v = {acc[mi][ni][jq * 4] * scale, acc[mi][ni][jq * 4 + 1] * scale, acc[mi][ni][jq * 4 + 2] * scale,
                                 acc[mi][ni][jq * 4 + 3] * scale};
                *reinterpret_cast<f32x4 *>(stage + b * LDF + a) = v;
            }
    // what the epilogue reads from memory (the old values of dx, and for DOT the other matrix) is requested before the barrier, so
    // that the loads are in flight while the staging tile fills
    constexpr int NP = RB_BI * RB_BT / 8 / 256;
    Frag8 old[NP], ot[NP];
    bool live[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int idx = q * 256 + t, b = idx / (RB_BI / 8), a = (idx % (RB_BI / 8)) * 8;
        live[q] = tok0 + b < p.tokens && i0 + a < p.in_f;   // in_f is a multiple of 8: a piece lies inside or outside
        if (live[q]) old[q].f4 = *reinterpret_cast<const f32x4 *>(p.dx + (int64_t)(tok0 + b) * p.lddx + i0 + a);
    }
    __syncthreads();
    if (DOT) {   // the accumulators are in LDS now: their registers take the other matrix's pieces
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int idx = q * 256 + t, b = idx / (RB_BI / 8), a = (idx % (RB_BI / 8)) * 8;
            if (live[q]) ot[q].f4 = *reinterpret_cast<const f32x4 *>(p.other + (int64_t)(tok0 + b) * p.ld_other + i0 + a);
        }
    }
    float dot = 0.0f;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int idx = q * 256 + t, b = idx / (RB_BI / 8), a = (idx % (RB_BI / 8)) * 8;
        if (live[q]) {
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(stage + b * LDF + a), hi = *reinterpret_cast<const f32x4 *>(stage + b * LDF + a + 4);
            if (DOT) {
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    dot = fmaf(lo[2 * e], __uint_as_float(ot[q].u[e] << 16), dot);
                    dot = fmaf(lo[2 * e + 1], __uint_as_float(ot[q].u[e] & 0xffff0000u), dot);
                    dot = fmaf(hi[2 * e], __uint_as_float(ot[q].u[2 + e] << 16), dot);
                    dot = fmaf(hi[2 * e + 1], __uint_as_float(ot[q].u[2 + e] & 0xffff0000u), dot);
                }
            }
            Frag8 nw;
            nw.u[0] = f32x2_to_bf16x2(__uint_as_float(old[q].u[0] << 16) + sval * lo[0], __uint_as_float(old[q].u[0] & 0xffff0000u) + sval * lo[1]);
            nw.u[1] = f32x2_to_bf16x2(__uint_as_float(old[q].u[1] << 16) + sval * lo[2], __uint_as_float(old[q].u[1] & 0xffff0000u) + sval * lo[3]);
            nw.u[2] = f32x2_to_bf16x2(__uint_as_float(old[q].u[2] << 16) + sval * hi[0], __uint_as_float(old[q].u[2] & 0xffff0000u) + sval * hi[1]);
            nw.u[3] = f32x2_to_bf16x2(__uint_as_float(old[q].u[3] << 16) + sval * hi[2], __uint_as_float(old[q].u[3] & 0xffff0000u) + sval * hi[3]);
            *reinterpret_cast<f32x4 *>(p.dx + (int64_t)(tok0 + b) * p.lddx + i0 + a) = nw.f4;
        }
    }
    if (DOT) {
        // the block's share of <src . R, other>: lanes, then waves, in a fixed order
        __shared__ float wsum[4];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (lane == 0) wsum[wave] = dot;
        __syncthreads();
        if (t == 0) p.dot_part[w] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
    }
}

// The same product on a tile of 64 features x 512 tokens with eight waves (one block per compute unit, two waves per SIMD).
// The hashing of R is what bounds these kernels on the vector ALU, and it is done once per block and stage whatever the
// number of tokens: a tile twice as long in tokens hashes half as much per matrix instruction.  A wave owns 64 tokens x 64
// features; R's tile is read by all waves, every wave reads its own part of the other operand's tile.  Used when the layer
// has enough such tiles to occupy the chip.
constexpr int RW_BI = 64, RW_BT = 512, RW_BK = 64, RW_THREADS = 512;
typedef OperandTile<RW_BI, RW_BK, K_CONT> RwTileR;
typedef OperandTile<RW_BT, RW_BK, K_CONT> RwTileS;
constexpr int RW_STAGE = RwTileR::LDS_ELEMS + RwTileS::LDS_ELEMS;   // elements of one pipeline stage in LDS
constexpr int RW_SP = RW_BT * RW_BK / 8 / RW_THREADS;                // 16-byte pieces of the other operand per thread and stage
static_assert(RW_BI * RW_BK / 8 == RW_THREADS, "one piece of R per thread and stage");

struct RwState {
    __amdgpu_buffer_rsrc_t rs_src;
    uint32_t soff[RW_SP];   // byte offset of the thread's pieces at stage 0 (BUFFER_OOB: token past the end)
    int pc8;                // contraction offset of the thread's pieces inside a stage
    int contraction;
    uint32_t first0, step, stage_step;   // R: first-round value of the thread's piece at stage 0, per contraction value, per stage
    int lds_r, lds_s;       // element offsets of the thread's pieces inside a stage (piece q of the other operand: + q * 64 rows)
};

__device__ __forceinline__ void rw_load_src(f32x4 (&rs)[RW_SP], const RwState &st, int stage)
{
    const uint32_t adv = (stage * RW_BK + st.pc8 < st.contraction) ? (uint32_t)(stage * RW_BK * 2) : BUFFER_OOB;
#pragma unroll
    for (int q = 0; q < RW_SP; ++q) rs[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(st.rs_src, (int)(st.soff[q] + adv), 0, 0));
}

__device__ __forceinline__ f32x4 rw_hash(const RwState &st, int stage)
{
    const uint32_t first = st.first0 + (uint32_t)stage * st.stage_step;
    uint32_t b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * st.step);
    Frag8 f;
#pragma unroll
    for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
    return f.f4;
}

// One stage: the matrix instructions of LDS buffer `cur`; between them the registers (holding the next stage) go to the
// other buffer (STORE) and are refilled with the stage after that (RELOAD).
template <bool STORE, bool RELOAD>
__device__ __forceinline__ void rw_stage(f32x16 (&acc)[2][2], const bf16_t *__restrict__ cur, bf16_t *__restrict__ oth, f32x4 (&rs)[RW_SP], f32x4 &rr,
                                         const RwState &st, int next, int wave, int lane)
{
    constexpr int KS = RW_BK / 16;
    const bf16_t *Rs = cur, *Ss = cur + RwTileR::LDS_ELEMS;
    bf16x8 fa[2][2], fb[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) fa[0][mi] = RwTileR::frag(Rs, mi * 32, 0, lane);
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) fb[0][ni] = RwTileS::frag(Ss, wave * 64 + ni * 32, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int c = ks & 1, n = c ^ 1;
#pragma unroll
        for (int q = 0; q < RW_SP; ++q)
            if (q % KS == ks) {
                if (STORE) *reinterpret_cast<f32x4 *>(oth + RwTileR::LDS_ELEMS + st.lds_s + q * 64 * RwTileS::LD) = rs[q];
                if (RELOAD) {
                    const uint32_t adv = (next * RW_BK + st.pc8 < st.contraction) ? (uint32_t)(next * RW_BK * 2) : BUFFER_OOB;
                    rs[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(st.rs_src, (int)(st.soff[q] + adv), 0, 0));
                }
            }
        if (ks == 0) {
            if (STORE) *reinterpret_cast<f32x4 *>(oth + st.lds_r) = rr;
            if (RELOAD) rr = rw_hash(st, next);
        }
        if (ks + 1 < KS) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) fa[n][mi] = RwTileR::frag(Rs, mi * 32, ks + 1, lane);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) fb[n][ni] = RwTileS::frag(Ss, wave * 64 + ni * 32, ks + 1, lane);
        }
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[c][mi], fb[c][ni], acc[mi][ni], 0, 0, 0);
    }
    __syncthreads();
}

template <bool DOT> __global__ __launch_bounds__(RW_THREADS, 1) void rbias_wide_kernel(RBiasParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    const int w = xcd_work_item(blockIdx.x, p.tiles_i * p.tiles_t);
    if (w >= p.tiles_i * p.tiles_t) return;
    const int i0 = (w % p.tiles_i) * RW_BI, tok0 = (w / p.tiles_i) * RW_BT;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5;
    const int prow = t >> 3, pc = t & 7;   // the thread's pieces: row prow (+ 64 q) of a tile, 16-byte chunk pc of the row
    RwState st;
    st.rs_src = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.dy), 0, (int)(((int64_t)(p.tokens - 1) * p.lddy + p.out_f) * 2), 0x00020000);
    st.pc8 = pc * 8;
    st.contraction = p.out_f;
#pragma unroll
    for (int q = 0; q < RW_SP; ++q) {
        const int tok = tok0 + q * 64 + prow;
        st.soff[q] = tok < p.tokens ? (uint32_t)(((int64_t)tok * p.lddy + pc * 8) * 2) : BUFFER_OOB;
    }
    st.step = p.sK * SQ5_N1;
    st.stage_step = (uint32_t)RW_BK * st.step;
    st.first0 = ((uint32_t)(i0 + prow) * p.sR + (uint32_t)(pc * 8) * p.sK) * SQ5_N1 + p.seed;
    st.lds_r = prow * RwTileR::LD + ((pc ^ RwTileR::swz(prow)) * 8);
    st.lds_s = prow * RwTileS::LD + ((pc ^ RwTileS::swz(prow)) * 8);   // the swizzle of row prow + 64 q is that of row prow

    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = zero16();
    const int nstage = (p.out_f + RW_BK - 1) / RW_BK;
    f32x4 rs[RW_SP], rr;
    {
        f32x4 rs0[RW_SP];
        rw_load_src(rs0, st, 0);
        rw_load_src(rs, st, 1);
        const f32x4 rr0 = rw_hash(st, 0);
        rr = rw_hash(st, 1);
#pragma unroll
        for (int q = 0; q < RW_SP; ++q) *reinterpret_cast<f32x4 *>(lds + RwTileR::LDS_ELEMS + st.lds_s + q * 64 * RwTileS::LD) = rs0[q];
        *reinterpret_cast<f32x4 *>(lds + st.lds_r) = rr0;
    }
    __syncthreads();
    int s = 0;
    for (; s + 2 < nstage; ++s) rw_stage<true, true>(acc, lds + (s & 1) * RW_STAGE, lds + ((s & 1) ^ 1) * RW_STAGE, rs, rr, st, s + 2, wave, lane);
    if (s + 1 < nstage) {
        rw_stage<true, false>(acc, lds + (s & 1) * RW_STAGE, lds + ((s & 1) ^ 1) * RW_STAGE, rs, rr, st, 0, wave, lane);
        ++s;
    }
    rw_stage<false, false>(acc, lds + (s & 1) * RW_STAGE, lds + ((s & 1) ^ 1) * RW_STAGE, rs, rr, st, 0, wave, lane);

    // dst += s * (2^-31 * acc), through LDS as fp32 so that every lane updates 8 consecutive features of a token's row
    const float sval = bf16_to_f32(*p.scale_bias);
    constexpr float scale = 4.656612873077392578125e-10f;
    constexpr int LDF = RW_BI + 4;
    float *stage = reinterpret_cast<float *>(smem_raw);
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const int b = wave * 64 + ni * 32 + r, a = mi * 32 + 8 * jq + 4 * g;
                const f32x4 v = {acc[mi][ni][jq * 4] * scale, acc[mi][ni][jq * 4 + 1] * scale, acc[mi][ni][jq * 4 + 2] * scale,
                                 acc[mi][ni][jq * 4 + 3] * scale};
                *reinterpret_cast<f32x4 *>(stage + b * LDF + a) = v;
            }
    constexpr int NP = RW_BI * RW_BT / 8 / RW_THREADS;
    Frag8 old[NP], ot[NP];
    bool live[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int b = q * 64 + prow, a = pc * 8;
        live[q] = tok0 + b < p.tokens && i0 + a < p.in_f;   // in_f is a multiple of 8: a piece lies inside or outside
        if (live[q]) old[q].f4 = *reinterpret_cast<const f32x4 *>(p.dx + (int64_t)(tok0 + b) * p.lddx + i0 + a);
    }
    __syncthreads();
    if (DOT) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = q * 64 + prow, a = pc * 8;
            if (live[q]) ot[q].f4 = *reinterpret_cast<const f32x4 *>(p.other + (int64_t)(tok0 + b) * p.ld_other + i0 + a);
        }
    }
    float dot = 0.0f;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int b = q * 64 + prow, a = pc * 8;
        if (live[q]) {
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(stage + b * LDF + a), hi = *reinterpret_cast<const f32x4 *>(stage + b * LDF + a + 4);
            if (DOT) {
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    dot = fmaf(lo[2 * e], __uint_as_float(ot[q].u[e] << 16), dot);
                    dot = fmaf(lo[2 * e + 1], __uint_as_float(ot[q].u[e] & 0xffff0000u), dot);
                    dot = fmaf(hi[2 * e], __uint_as_float(ot[q].u[2 + e] << 16), dot);
                    dot = fmaf(hi[2 * e + 1], __uint_as_float(ot[q].u[2 + e] & 0xffff0000u), dot);
                }
            }
            Frag8 nw;
            nw.u[0] = f32x2_to_bf16x2(__uint_as_float(old[q].u[0] << 16) + sval * lo[0], __uint_as_float(old[q].u[0] & 0xffff0000u) + sval * lo[1]);
            nw.u[1] = f32x2_to_bf16x2(__uint_as_float(old[q].u[1] << 16) + sval * lo[2], __uint_as_float(old[q].u[1] & 0xffff0000u) + sval * lo[3]);
            nw.u[2] = f32x2_to_bf16x2(__uint_as_float(old[q].u[2] << 16) + sval * hi[0], __uint_as_float(old[q].u[2] & 0xffff0000u) + sval * hi[1]);
            nw.u[3] = f32x2_to_bf16x2(__uint_as_float(old[q].u[3] << 16) + sval * hi[2], __uint_as_float(old[q].u[3] & 0xffff0000u) + sval * hi[3]);
            *reinterpret_cast<f32x4 *>(p.dx + (int64_t)(tok0 + b) * p.lddx + i0 + a) = nw.f4;
        }
    }
    if (DOT) {
        __shared__ float wsum[RW_THREADS / 64];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (lane == 0) wsum[wave] = dot;
        __syncthreads();
        if (t == 0) p.dot_part[w] = ((wsum[0] + wsum[1]) + (wsum[2] + wsum[3])) + ((wsum[4] + wsum[5]) + (wsum[6] + wsum[7]));
    }
}

// out[0] = part[0] + ... + part[n - 1], in a fixed order (one block)
__global__ __launch_bounds__(256) void rbias_sum_kernel(float *__restrict__ out, const float *__restrict__ part, int n)
{
    __shared__ float sh[256];
    float v = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) v += part[i];
    sh[threadIdx.x] = v;
    __syncthreads();
    for (int h = 128; h >= 1; h >>= 1) {
        if ((int)threadIdx.x < h) sh[threadIdx.x] += sh[threadIdx.x + h];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = sh[0];
}

// other / dot_part / dscale: NULL, or the matrix the product is reduced against, room for one float per tile, and where the sum goes
static int rbias_add(void *dst, int64_t ld_dst, int64_t cols, const void *src, int64_t ld_src, int64_t contraction, uint32_t sR, uint32_t sK,
                     const void *scale_bias, const rdb_linear_desc *d, hipStream_t s, const void *other = nullptr, int64_t ld_other = 0,
                     float *dot_part = nullptr, float *dscale = nullptr)
{
    if (d->act_dtype != RDB_BF16 || d->coef_dtype != RDB_BF16 || d->coef_rows == 0 || !scale_bias) return RDB_E_UNSUPPORTED;
    if (d->in_f % 8 || d->out_f % 8 || d->tokens < 1 || d->in_f < 1 || d->out_f < 1) return RDB_E_UNSUPPORTED;
    if (ld_src % 8 || ld_dst % 8 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens * ld_src >= (1ll << 29) || d->tokens * ld_dst >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    RBiasParams p;
    p.dy = (const bf16_t *)src;
    p.scale_bias = (const bf16_t *)scale_bias;
    p.dx = (bf16_t *)dst;
    p.lddy = ld_src;
    p.lddx = ld_dst;
    p.tokens = (int)d->tokens;
    p.in_f = (int)cols;
    p.out_f = (int)contraction;
    p.tiles_i = (int)cdiv(cols, RB_BI);
    p.tiles_t = (int)cdiv(d->tokens, RB_BT);
    p.sR = sR;
    p.sK = sK;
    p.seed = d->seed;
    p.other = (const bf16_t *)other;
    p.ld_other = ld_other;
    p.dot_part = dot_part;
    if (other && (ld_other % 8 || ((uintptr_t)other & 15) || d->tokens * ld_other >= (1ll << 29) || !dot_part || !dscale)) return RDB_E_UNSUPPORTED;
    // tiles of 512 tokens when they give at least every other compute unit a block (half the hashing per product: measured
    // ahead from there on; 8192 tokens x 768 features, contraction 3072: 83 -> 67 us), tiles of 256 tokens otherwise
    const int wide_items = (int)(cdiv(cols, RW_BI) * cdiv(d->tokens, RW_BT));
    if (wide_items * 2 >= num_compute_units()) {
        p.tiles_i = (int)cdiv(cols, RW_BI);
        p.tiles_t = (int)cdiv(d->tokens, RW_BT);
        const size_t wsmem = (size_t)2 * RW_STAGE * sizeof(bf16_t);
        static_assert((size_t)RW_BT * (RW_BI + 4) * sizeof(float) <= (size_t)2 * RW_STAGE * sizeof(bf16_t), "the fp32 staging tile fits the pipeline's LDS");
        if (!other) {
            if (int rl = reserve_lds(reinterpret_cast<const void *>(rbias_wide_kernel<false>), wsmem, "rbias_wide_kernel")) return rl;
            rbias_wide_kernel<false><<<xcd_grid_size(wide_items), RW_THREADS, wsmem, s>>>(p);
            return check_launch("rbias_wide_kernel");
        }
        if (int rl = reserve_lds(reinterpret_cast<const void *>(rbias_wide_kernel<true>), wsmem, "rbias_wide_kernel<dot>")) return rl;
        rbias_wide_kernel<true><<<xcd_grid_size(wide_items), RW_THREADS, wsmem, s>>>(p);
        if (int rc = check_launch("rbias_wide_kernel<dot>")) return rc;
        rbias_sum_kernel<<<1, 256, 0, s>>>(dscale, dot_part, wide_items);
        return check_launch("rbias_sum_kernel");
    }
    size_t smem = engine_smem<RB_BI, RB_BT, RB_BK, K_CONT, K_CONT>();
    const size_t stage = (size_t)RB_BT * (RB_BI + 4) * sizeof(float);
    if (smem < stage) smem = stage;
    if (!other) return launch_engine(rbias_add_kernel<false>, p, p.tiles_i * p.tiles_t, smem, s, "rbias_add_kernel");
    if (int rc = launch_engine(rbias_add_kernel<true>, p, p.tiles_i * p.tiles_t, smem, s, "rbias_add_kernel<dot>")) return rc;
    rbias_sum_kernel<<<1, 256, 0, s>>>(dscale, dot_part, p.tiles_i * p.tiles_t);
    return check_launch("rbias_sum_kernel");
}

// floats of scratch for the tiles' shares of the scale's gradient
int64_t linear_dx_rbias_dot_floats(const rdb_linear_desc *d) { return cdiv(d->in_f, RB_BI) * cdiv(d->tokens, RB_BT); }

// dx += s * dy . R and d s = <dy . R, x> in one pass over dy . R
int linear_dx_rbias_add_dscale(void *dx, int64_t lddx, float *dscale, float *dot_part, const void *dy, int64_t lddy, const void *x, int64_t ldx,
                               const void *scale_bias, const rdb_linear_desc *d, hipStream_t s)
{
    return rbias_add(dx, lddx, d->in_f, dy, lddy, d->out_f, 1u, (uint32_t)d->in_f, scale_bias, d, s, x, ldx, dot_part, dscale);
}

// dx += s * dy . R on the launch stream, after the kernels that wrote dx.  Returns RDB_E_UNSUPPORTED (without setting an
// error) when the request does not fit.
int linear_dx_rbias_add(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *scale_bias, const rdb_linear_desc *d, hipStream_t s)
{
    return rbias_add(dx, lddx, d->in_f, dy, lddy, d->out_f, 1u, (uint32_t)d->in_f, scale_bias, d, s);
}

// y += s * x . R^T on the launch stream, after the kernels that wrote y; same conditions.
int linear_fwd_rbias_add(void *y, int64_t ldy, const void *x, int64_t ldx, const void *scale_bias, const rdb_linear_desc *d, hipStream_t s)
{
    return rbias_add(y, ldy, d->out_f, x, ldx, d->in_f, (uint32_t)d->in_f, 1u, scale_bias, d, s);
}

}  // namespace rdb
