// bf16 MFMA tile engine for gfx950 shared by the optimised fused-linear kernels.
//
// A 256-thread block (4 waves as 2 x 2) accumulates a BM x BN tile D[m][n] += sum_k A[m][k] * B[n][k] in fp32 with
// v_mfma_f32_32x32x16_bf16.  Each operand comes from global memory in one of two layouts:
//   K_CONT : src[row * ld + k]   the contraction index is contiguous (x for y = x.W^T, dy for dx = dy.W, C for z.C^T)
//   M_CONT : src[k * ld + row]   the tile row index is contiguous     (dy and x for dW = dy^T.x, C for dy.C)
// Both are staged through LDS with straight 16-byte copies.  K_CONT fragments are read with ds_read_b128; M_CONT
// fragments with two ds_read_b64_tr_b16 (the LDS transpose read of gfx950), which hands lane c of each 16-lane group
// column c of a 4 (k) x 16 (row) patch, i.e. exactly the k-contiguous fragment the matrix core wants.
//
// Pipeline: LDS is double buffered with one barrier per stage; global loads run DA (operand A) or DB (operand B) stages
// further ahead in registers, so that enough bytes are in flight per compute unit to cover HBM latency.
#pragma once

#include "rdb_common.hpp"
#include "rdb_tile.hpp"

namespace rdb {

typedef short s16x4 __attribute__((ext_vector_type(4)));

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Byte offset that lies outside every buffer the tile engine reads (operands are smaller than 2^30 bytes): a buffer load
// at this offset fails the hardware bounds check and returns zeros, without a branch and without touching memory.  Two of
// them, or one plus any in-range offset, still add up to an out-of-range offset below 2^32.
constexpr uint32_t BUFFER_OOB = 0x40000000u;

enum OperandLayout { K_CONT = 0, M_CONT = 1 };

union Frag8 {
    bf16x8 v;
    s16x4 h[2];
    uint32_t u[4];
    f32x4 f4;
};

// One operand of the tile engine.  ROWS = tile rows (BM or BN), BK = contraction depth per stage.
template <int ROWS, int BK, int LAYOUT> struct OperandTile {
    // LDS layout, chosen so that the 16-byte copy stores and the fragment reads are both free of bank conflicts
    // (64 banks of 4 bytes; a 128-bit access is served 16 lanes at a time, a 64-bit one 32 lanes at a time):
    // K_CONT: rows of BK = 64 elements (128 bytes) without padding, 16-byte chunk c of row r stored at chunk position
    //         c ^ ((r >> 1) & 7).  A store phase covers two whole rows (256 contiguous bytes); a read phase takes one
    //         chunk from each of 16 consecutive rows, which the swizzle spreads over all 16 chunk positions of a row pair.
    // M_CONT: rows (one per k) of ROWS elements plus 64 bytes of padding, so the 4 k-rows one ds_read_b64_tr_b16 phase
    //         touches (64 bytes each) tile the 64 banks exactly.
    // K_CONT with BK = 128: rows of 256 bytes, chunk c of row r at position c ^ (r & 15): a read phase (one chunk from each
    //         of 16 consecutive rows) and a store phase (one whole row) both touch all 16 chunk positions once.
    static_assert(LAYOUT == M_CONT || BK == 64 || BK == 128, "the swizzled K_CONT layout is laid out for rows of 64 or 128 elements");
    __device__ static __forceinline__ int swz(int row) { return BK == 64 ? ((row >> 1) & 7) : (row & 15); }
    static constexpr int PAD = (LAYOUT == K_CONT) ? 0 : 32;
    static constexpr int LAYOUT_ID = LAYOUT;
    static constexpr int LD = (LAYOUT == K_CONT) ? (BK + PAD) : (ROWS + PAD);     // LDS row stride, elements
    static constexpr int LDS_ELEMS = (LAYOUT == K_CONT) ? ROWS * LD : BK * LD;    // per stage
    static constexpr int PIECES = ROWS * BK / 8;                                   // 16-byte pieces per stage
    static constexpr int PER_THREAD = (PIECES + 255) / 256;
    static_assert(PIECES % 256 == 0, "operand stage must split evenly over 256 threads");

    // Per-thread description of the pieces it copies from global memory: byte offset of each piece at stage 0, BUFFER_OOB
    // when its tile row lies outside the matrix.  Built once, before the loop.
    struct Pieces {
        uint32_t off[PER_THREAD];
    };
    // K_CONT: the contraction offset of a thread's pieces inside a stage is the same for all of them (256 % (BK/8) == 0).
    __device__ static __forceinline__ int thread_kk() { return (threadIdx.x % (BK / 8)) * 8; }
    __device__ static __forceinline__ Pieces pieces(int64_t ld, int row0, int nrows, int k_begin)
    {
        Pieces q;
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int idx = p * 256 + t;
            int row, k;
            if (LAYOUT == K_CONT) {
                row = row0 + idx / (BK / 8);
                k = (idx % (BK / 8)) * 8;
            } else {
                k = idx / (ROWS / 8);
                row = row0 + (idx % (ROWS / 8)) * 8;
            }
            const uint32_t elem = (LAYOUT == K_CONT) ? (uint32_t)(row * ld) + k_begin + k : (uint32_t)((k_begin + k) * ld) + row;
            q.off[p] = row < nrows ? elem * 2u : BUFFER_OOB;
        }
        return q;
    }

    // Global -> register for piece p; `adv` is the byte offset of the stage relative to stage 0, or BUFFER_OOB.  A buffer
    // load: pieces outside the matrix carry an out-of-range offset and come back as zeros.  The host guarantees that the
    // contiguous axis is a multiple of 8, so a 16-byte piece is entirely inside or outside.
    __device__ static __forceinline__ void load_piece(f32x4 &reg, __amdgpu_buffer_rsrc_t rsrc, const Pieces &q, int p, uint32_t adv)
    {
        reg = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(q.off[p] + adv), 0, 0));
    }

    // Registers -> LDS stage.
    __device__ static __forceinline__ void store_piece(bf16_t *__restrict__ lds, const f32x4 &reg, int p)
    {
        const int idx = p * 256 + threadIdx.x;
        int off;
        if (LAYOUT == K_CONT) {
            const int row = idx / (BK / 8), c = idx % (BK / 8);
            off = row * LD + ((c ^ swz(row)) * 8);
        } else {
            off = (idx / (ROWS / 8)) * LD + (idx % (ROWS / 8)) * 8;
        }
        *reinterpret_cast<f32x4 *>(lds + off) = reg;
    }
    __device__ static __forceinline__ void store(bf16_t *__restrict__ lds, const f32x4 (&regs)[PER_THREAD])
    {
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) store_piece(lds, regs[p], p);
    }

    // Fragment of the 32-row block starting at tile row `rb` for k-step ks (16 wide) of the stage:
    // lane (r = lane % 32, g = lane / 32) gets k = ks*16 + g*8 .. +7 of row rb + r.
    __device__ static __forceinline__ bf16x8 frag(const bf16_t *__restrict__ lds, int rb, int ks, int lane)
    {
        Frag8 f;
        const int r = lane & 31, g = lane >> 5;
        if (LAYOUT == K_CONT) {
            // rb is a multiple of 32, so the swizzle depends on the lane only
            f.v = *reinterpret_cast<const bf16x8 *>(lds + (rb + r) * LD + (((ks * 2 + g) ^ swz(r)) * 8));
        } else {
            // 16-lane group q = (lane / 16) & 1 covers rows rb + 16q .. +15; source lane s of the group addresses
            // k = kb + s / 4, rows 4*(s % 4) .. +3; the result lane c receives rows' column c for k = kb .. kb+3.
            const int s = lane & 15, q = (lane >> 4) & 1;
            const int kb = ks * 16 + g * 8;
            const bf16_t *p = lds + (kb + (s >> 2)) * LD + rb + q * 16 + (s & 3) * 4;
            f.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(p));
            f.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(p + 4 * LD));
        }
        return f.v;
    }
};

// ----------------------------------------------------------------------------------------------- work distribution
// The 8 accelerator dies (XCDs) of the chip each have their own L2 and receive workgroups round-robin by linear block id.
// Work items that read the same operand tiles should therefore sit on one die and run at the same time: item w of `total`
// (neighbours in w share operands) goes to block id  (w % per_die) * 8 + w / per_die,  i.e. a block decodes
//   w = (block % 8) * per_die + block / 8,   per_die = ceil(total / 8);   w >= total means the block has nothing to do.
__device__ __forceinline__ int xcd_work_item(int block, int total)
{
    const int per_die = (total + 7) >> 3;
    return (block & 7) * per_die + (block >> 3);
}
inline int xcd_grid_size(int total) { return ((total + 7) / 8) * 8; }

// ----------------------------------------------------------------------------------------------- operand providers
// A provider fills the registers of one pipeline stage: load(regs, k0) with k0 the stage's first contraction index.

// Operand read from global memory through a buffer resource (the operand must be smaller than 2^31 bytes).
// extent: number of elements from `src` that may be read (last row's end).
template <int ROWS, int BK, int LAYOUT> struct GlobalOperand {
    typedef OperandTile<ROWS, BK, LAYOUT> Tile;
    const bf16_t *src;
    int64_t ld;
    int row0, nrows, klim;  // klim: first contraction index that must read as zero
    int64_t extent;
    typename Tile::Pieces q;
    __amdgpu_buffer_rsrc_t rsrc;
    int k_begin, kk;
    __device__ __forceinline__ void init(int kb)
    {
        k_begin = kb;
        kk = Tile::thread_kk();
        q = Tile::pieces(ld, row0, nrows, kb);
        // M_CONT: contraction indices are rows of the source, so clipping the buffer at row klim makes the hardware bounds
        // check zero everything from klim on.  K_CONT clips per thread in load_piece().
        int64_t bytes = extent * 2;
        if (LAYOUT == M_CONT && (int64_t)klim * ld * 2 < bytes) bytes = (int64_t)klim * ld * 2;
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(src), 0, (int)bytes, 0x00020000);
    }
    __device__ __forceinline__ void load_piece(f32x4 &reg, int p, int stage) const
    {
        // one offset per stage (the same expression for every piece: computed once), one add per piece
        uint32_t adv;
        if (LAYOUT == K_CONT)
            adv = (k_begin + stage * BK + kk < klim) ? (uint32_t)(stage * BK * 2) : BUFFER_OOB;
        else   // stages that begin at or past klim (round-up of the trip count, prefetch past the end) must not depend on the
               // 32-bit product below staying out of bounds: with a huge leading dimension it could wrap back into the buffer
            adv = (k_begin + stage * BK < klim) ? (uint32_t)stage * (uint32_t)(BK * 2) * (uint32_t)ld : BUFFER_OOB;
        Tile::load_piece(reg, rsrc, q, p, adv);
    }
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int stage) const
    {
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p) load_piece(regs[p], p, stage);
    }
};

// Operand generated by the noise hash, tile rows = noise rows (tensor element index), contraction = coefficient index:
// element (row, k) = 2^31 * noise(PRIME*(row0 + row) + k) as bf16 (callers fold the 2^-31 into their epilogue).
template <int ROWS, int BK> struct NoiseOperandRowsAreElements {
    typedef OperandTile<ROWS, BK, K_CONT> Tile;
    int row0;
    uint32_t seed;
    int k_begin;
    __device__ __forceinline__ void init(int kb) { k_begin = kb; }
    __device__ __forceinline__ void load_piece(f32x4 &reg, int p, int stage) const
    {
        const int idx = p * 256 + threadIdx.x, k0 = k_begin + stage * BK;
        const int row = row0 + idx / (BK / 8), k = k0 + (idx % (BK / 8)) * 8;
        const uint32_t first = (uint32_t)row * PN1 + (uint32_t)k * SQ5_N1 + seed;
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * SQ5_N1);
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

// Same noise, tile rows = coefficient index, contraction = element index: element (row, k) = 2^31 * noise(PRIME*k + row0 + row).
template <int ROWS, int BK> struct NoiseOperandRowsAreCoefs {
    typedef OperandTile<ROWS, BK, K_CONT> Tile;
    int row0;
    uint32_t seed;
    int k_begin;
    __device__ __forceinline__ void init(int kb) { k_begin = kb; }
    __device__ __forceinline__ void load_piece(f32x4 &reg, int p, int stage) const
    {
        const int idx = p * 256 + threadIdx.x, k0 = k_begin + stage * BK;
        const int row = row0 + idx / (BK / 8), k = k0 + (idx % (BK / 8)) * 8;
        const uint32_t first = (uint32_t)k * PN1 + (uint32_t)row * SQ5_N1 + seed;
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * PN1);
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

// One pipeline stage: multiplies the LDS buffer `cur` into the accumulators while, slice by slice between the MFMAs, the
// registers `ra`/`rb` (holding the stage after this one) go to the idle buffer `oth` and are refilled with stages
// next_a / next_b.  The copy work and the next k-step's fragment reads are paced against the MFMAs with scheduling
// groups: every MFMA is followed by a fixed number of memory instructions, so the vector-memory and LDS pipes run in the
// shadow of the matrix pipe.
// STORE / RELOAD switch the copy work off for the stages at the end of the loop whose successors lie past the end.
template <int BK, int MI, int NI, bool STORE, bool RELOAD, class PA, class PB>
__device__ __forceinline__ void pipeline_stage(f32x16 (&acc)[MI][NI], const bf16_t *__restrict__ cur, bf16_t *__restrict__ oth,
                                               f32x4 (&ra)[PA::Tile::PER_THREAD], f32x4 (&rb)[PB::Tile::PER_THREAD], const PA &pa, const PB &pb,
                                               int next_a, int next_b, int wm, int wn, int lane)
{
    typedef typename PA::Tile TA;
    typedef typename PB::Tile TB;
    constexpr int KS = BK / 16;
    constexpr int FRAG_OPS = (MI * (TA::LAYOUT_ID == M_CONT ? 2 : 1)) + (NI * (TB::LAYOUT_ID == M_CONT ? 2 : 1));
    constexpr int COPY_OPS = ((STORE ? 1 : 0) + (RELOAD ? 1 : 0)) * ((TA::PER_THREAD + TB::PER_THREAD + KS - 1) / KS);
    constexpr int MEM_PER_MFMA = (FRAG_OPS + COPY_OPS + MI * NI - 1) / (MI * NI);
    const bf16_t *As = cur, *Bs = cur + TA::LDS_ELEMS;
    bf16x8 fa[2][MI], fb[2][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) fa[0][mi] = TA::frag(As, wm * MI * 32 + mi * 32, 0, lane);
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) fb[0][ni] = TB::frag(Bs, wn * NI * 32 + ni * 32, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int c = ks & 1, n = c ^ 1;
#pragma unroll
        for (int p = 0; p < TA::PER_THREAD; ++p)
            if (p % KS == ks) {
                if (STORE) TA::store_piece(oth, ra[p], p);
                if (RELOAD) pa.load_piece(ra[p], p, next_a);
            }
#pragma unroll
        for (int p = 0; p < TB::PER_THREAD; ++p)
            if ((p + TA::PER_THREAD) % KS == ks) {
                if (STORE) TB::store_piece(oth + TA::LDS_ELEMS, rb[p], p);
                if (RELOAD) pb.load_piece(rb[p], p, next_b);
            }
        if (ks + 1 < KS) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) fa[n][mi] = TA::frag(As, wm * MI * 32 + mi * 32, ks + 1, lane);
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) fb[n][ni] = TB::frag(Bs, wn * NI * 32 + ni * 32, ks + 1, lane);
        }
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[c][mi], fb[c][ni], acc[mi][ni], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < MI * NI; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x090, MEM_PER_MFMA, 0);  // then vector-memory / LDS instructions
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
}

// Main loop of the tile engine over `nstage` stages of BK starting at contraction index k_begin.
// DA / DB (1, 2 or 4): how many stages ahead of the LDS copy the registers of operand A / B are loaded.
// `lds` must hold 2 * (PA::Tile::LDS_ELEMS + PB::Tile::LDS_ELEMS) elements.  On return every wave has passed a barrier
// after its last LDS read, so the caller may reuse `lds` at once.  The stage count is rounded up to a multiple of the
// unrolled trip (the extra stages lie past klim and read as zeros), so the loop body has a single exit; the last trip is
// peeled and does no reloads.
// WM: waves along the A rows (2: 2 x 2 waves, 1: 1 x 4, 4: 4 x 1); a wave owns (BM / WM) x (BN / (4 / WM)) of the tile.
template <int BM, int BN, int BK, int DA, int DB, int WM = 2, class PA, class PB>
__device__ __forceinline__ void gemm_mainloop(f32x16 (&acc)[BM / (32 * WM)][BN / (128 / WM)], bf16_t *__restrict__ lds, PA &pa, PB &pb,
                                              int k_begin, int nstage)
{
    typedef typename PA::Tile TA;
    typedef typename PB::Tile TB;
    static_assert((DA == 1 || DA == 2 || DA == 4) && (DB == 1 || DB == 2 || DB == 4), "prefetch depth must be 1, 2 or 4");
    static_assert(WM == 1 || WM == 2 || WM == 4, "4 waves as 1x4, 2x2 or 4x1");
    constexpr int WN = 4 / WM, MI = BM / (32 * WM), NI = BN / (32 * WN);
    static_assert(MI * 32 * WM == BM && NI * 32 * WN == BN, "tile must split into 32-row blocks per wave");
    constexpr int STAGE = TA::LDS_ELEMS + TB::LDS_ELEMS;
    constexpr int TRIP = (DA == 4 || DB == 4) ? 4 : 2;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, wm = wave / WN, wn = wave % WN;
    if (nstage <= 0) return;
    RDB_STAMP(0);
    pa.init(k_begin);
    pb.init(k_begin);

    // registers of stage j live in slot j % D; stage 0 goes through a set of its own straight to LDS
    f32x4 ra[DA][TA::PER_THREAD], rb[DB][TB::PER_THREAD];
    {
        f32x4 ra0[TA::PER_THREAD], rb0[TB::PER_THREAD];
        pa.load(ra0, 0);
        pb.load(rb0, 0);
#pragma unroll
        for (int j = 1; j <= DA; ++j) pa.load(ra[j % DA], j);
#pragma unroll
        for (int j = 1; j <= DB; ++j) pb.load(rb[j % DB], j);
        TA::store(lds, ra0);
        TB::store(lds + TA::LDS_ELEMS, rb0);
    }
    __syncthreads();
    RDB_STAMP(1);

    const int nround = (nstage + TRIP - 1) / TRIP * TRIP;
    int s = 0;
    for (; s + TRIP < nround; s += TRIP) {
#pragma unroll
        for (int u = 0; u < TRIP; ++u) {
            // stage s+u is in LDS buffer u % 2; slot (u+1) % D holds stage s+u+1 and is refilled with stage s+u+1+D
            bf16_t *cur = lds + (u & 1) * STAGE, *oth = lds + ((u & 1) ^ 1) * STAGE;
            pipeline_stage<BK, MI, NI, true, true>(acc, cur, oth, ra[(u + 1) % DA], rb[(u + 1) % DB], pa, pb, s + u + 1 + DA, s + u + 1 + DB, wm,
                                                   wn, lane);
        }
    }
    // last trip: everything it would reload lies past the end (a hashed operand would hash for nothing), and its last
    // stage has nothing left to hand to LDS
#pragma unroll
    for (int u = 0; u < TRIP; ++u) {
        bf16_t *cur = lds + (u & 1) * STAGE, *oth = lds + ((u & 1) ^ 1) * STAGE;
        if (u + 1 < TRIP)
            pipeline_stage<BK, MI, NI, true, false>(acc, cur, oth, ra[(u + 1) % DA], rb[(u + 1) % DB], pa, pb, 0, 0, wm, wn, lane);
        else
            pipeline_stage<BK, MI, NI, false, false>(acc, cur, oth, ra[(u + 1) % DA], rb[(u + 1) % DB], pa, pb, 0, 0, wm, wn, lane);
    }
    RDB_STAMP(2);
}

// Writes the block's BM x BN accumulator tile D[a][b] as bf16 to out[(b0 + b) * ld + a0 + a] (rows of `out` run along a),
// v = acc * scale (+ bias[a0 + a]).  The tile is staged through LDS (BN x (BM + 8) elements) so that the global stores are
// 16 bytes wide and contiguous along each row.  Needs a0, na, ld multiples of 8 and a 16-byte aligned `out`.
// All 256 threads must call; `lds` must be free on entry (the main loop ends with a barrier) and is free again on return.
template <int BM, int BN, int WM = 2>
__device__ __forceinline__ void store_tile_bf16(const f32x16 (&acc)[BM / (32 * WM)][BN / (128 / WM)], bf16_t *__restrict__ lds,
                                                bf16_t *__restrict__ out, int64_t ld, int a0, int na, int b0, int nb, float scale,
                                                const bf16_t *__restrict__ bias)
{
    constexpr int WN = 4 / WM, MI = BM / (32 * WM), NI = BN / (32 * WN), LDS_LD = BM + 8;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave / WN, wn = wave % WN;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
            const int a = wm * MI * 32 + mi * 32 + 8 * jq + 4 * g;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e) bv[e] = (a0 + a + e < na) ? bf16_to_f32(bias[a0 + a + e]) : 0.0f;
            }
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int b = wn * NI * 32 + ni * 32 + r;
                store4<bf16_t>(lds + b * LDS_LD + a, acc[mi][ni][jq * 4 + 0] * scale + bv[0], acc[mi][ni][jq * 4 + 1] * scale + bv[1],
                               acc[mi][ni][jq * 4 + 2] * scale + bv[2], acc[mi][ni][jq * 4 + 3] * scale + bv[3]);
            }
        }
    __syncthreads();
    constexpr int PIECES = BM * BN / 8;
#pragma unroll
    for (int p = 0; p < PIECES / 256; ++p) {
        const int idx = p * 256 + t;
        const int b = idx / (BM / 8), a = (idx % (BM / 8)) * 8;
        if (b0 + b < nb && a0 + a < na)
            *reinterpret_cast<f32x4 *>(out + (int64_t)(b0 + b) * ld + a0 + a) = *reinterpret_cast<const f32x4 *>(lds + b * LDS_LD + a);
    }
    __syncthreads();
}

// Accumulators -> bf16 in MFMA-fragment order, for a consumer that keeps this matrix in registers as the "b" operand
// (rdb_stationary.hpp): 32 rows b by 16 columns a form one k-step of 1024 bytes, lane (b % 32, half) holding 8 columns:
//   element (b, a) -> ((b / 32) * ksteps + a / 16) * 512 + ((a / 8) % 2 * 32 + b % 32) * 8 + a % 8.
// Columns up to na and rows up to nb are written (pass them rounded up to the padding the consumer reads: the accumulators
// there are zeros).  Needs a0 a multiple of 8 and b0 of 32; `out` 16-byte aligned.
template <int BM, int BN, int WM = 2>
__device__ __forceinline__ void store_tile_bf16_frag(const f32x16 (&acc)[BM / (32 * WM)][BN / (128 / WM)], bf16_t *__restrict__ lds,
                                                     bf16_t *__restrict__ out, int ksteps, int a0, int na, int b0, int nb, float scale)
{
    constexpr int WN = 4 / WM, MI = BM / (32 * WM), NI = BN / (32 * WN), LDS_LD = BM + 8;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave / WN, wn = wave % WN;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
            const int a = wm * MI * 32 + mi * 32 + 8 * jq + 4 * g;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int b = wn * NI * 32 + ni * 32 + r;
                store4<bf16_t>(lds + b * LDS_LD + a, acc[mi][ni][jq * 4 + 0] * scale, acc[mi][ni][jq * 4 + 1] * scale,
                               acc[mi][ni][jq * 4 + 2] * scale, acc[mi][ni][jq * 4 + 3] * scale);
            }
        }
    __syncthreads();
    constexpr int PIECES = BM * BN / 8;
#pragma unroll
    for (int p = 0; p < PIECES / 256; ++p) {
        const int idx = p * 256 + t;
        const int b = idx % BN, a = (idx / BN) * 8;   // neighbouring lanes: neighbouring rows of one 8-column piece, 16 bytes apart in `out`
        const int gb = b0 + b, ga = a0 + a;
        if (gb < nb && ga < na)
            *reinterpret_cast<f32x4 *>(out + ((int64_t)(gb >> 5) * ksteps + (ga >> 4)) * 512 + (((ga >> 3) & 1) * 32 + (gb & 31)) * 8) =
                *reinterpret_cast<const f32x4 *>(lds + b * LDS_LD + a);
    }
    __syncthreads();
}

// ----------------------------------------------------------------------------------------------- host side helpers
// Dynamic LDS of an engine kernel: the two pipeline stages, or the bf16 output staging tile if that is larger.
template <int BM, int BN, int BK, int LA, int LB> inline size_t engine_smem()
{
    const size_t stages = 2 * (OperandTile<BM, BK, LA>::LDS_ELEMS + OperandTile<BN, BK, LB>::LDS_ELEMS) * sizeof(bf16_t);
    const size_t store = (size_t)BN * (BM + 8) * sizeof(bf16_t);
    return stages > store ? stages : store;
}

// Launches an engine kernel over `items` work items (one 256-thread block each, XCD-aware numbering).
template <class K, class P> inline int launch_engine(K kernel, const P &p, int items, size_t smem, hipStream_t s, const char *name)
{
    if (int rl = reserve_lds(reinterpret_cast<const void *>(kernel), smem, name)) return rl;
    kernel<<<xcd_grid_size(items), 256, smem, s>>>(p);
    return check_launch(name);
}

}  // namespace rdb
