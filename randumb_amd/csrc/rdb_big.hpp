// Large-tile, persistent form of the bf16 tile engine, for the three dense products of the factored algorithm when the
// coefficient dimension is long (k > 256):  y = z . C^T,  t = dy . C,  dC = dy^T . z.
//
// A 128 x 128 tile moves 64 bytes through a compute unit's vector-memory path per clock of matrix work, which is all that
// path delivers; a 256 x 256 tile needs half of that.  One 256-thread block per compute unit (four waves, one per SIMD, each
// owning 128 x 128 or 128 x 64 of the tile in up to 256 accumulator registers) walks over a list of tiles: while the
// finished tile leaves through LDS, the first stage of the block's next tile is already on its way from memory, so a tile
// costs its matrix work and little else.  The stage pipeline is the engine's (pipeline_stage of rdb_gemm.hpp).
//
// Operands come as K_CONT / M_CONT matrices (GlobalOperand) or in MFMA fragment order (FragOperand below: the transposed
// copies of z and C that the projection leaves in the state, and z itself), which passes through LDS as a straight copy.
#pragma once
#include "rdb_direct.hpp"

namespace rdb {

constexpr int F_CONT = 2;   // third operand layout: fragment order (frag_index of rdb_direct.hpp)

// LDS tile of a fragment-ordered operand: the image of the source, row block after row block, k-step after k-step; a
// fragment read is 64 lanes x 16 consecutive bytes.  BK = 64: a stage is 4 k-steps, i.e. 4 KB per row block.
template <int ROWS, int BK> struct FragTile {
    static_assert(BK == 64 && ROWS % 32 == 0, "a stage of a fragment-ordered operand is 4 k-steps of each 32-row block");
    static constexpr int LAYOUT_ID = F_CONT;
    static constexpr int KS = BK / 16;
    static constexpr int LDS_ELEMS = ROWS * BK;
    static constexpr int PER_THREAD = ROWS / 32;   // piece p of thread t: row block p, k-step t / 64, lane t % 64
    __device__ static __forceinline__ void store_piece(bf16_t *__restrict__ lds, const f32x4 &reg, int p)
    {
        *reinterpret_cast<f32x4 *>(lds + (p * 256 + (int)threadIdx.x) * 8) = reg;
    }
    __device__ static __forceinline__ void store(bf16_t *__restrict__ lds, const f32x4 (&regs)[PER_THREAD])
    {
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) store_piece(lds, regs[p], p);
    }
    __device__ static __forceinline__ bf16x8 frag(const bf16_t *__restrict__ lds, int rb, int ks, int lane)
    {
        return *reinterpret_cast<const bf16x8 *>(lds + ((rb >> 5) * KS + ks) * 512 + lane * 8);
    }
};

// Provider of a fragment-ordered matrix with `ksteps` k-steps per row block and `nrb` row blocks; the tile starts at row block
// rb0.  Row blocks past the end and k-steps from klim_steps on read as zeros (the buffer bounds check).
template <int ROWS, int BK> struct FragOperand {
    typedef FragTile<ROWS, BK> Tile;
    const bf16_t *src;
    int ksteps, nrb, rb0, klim_steps;
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t off[Tile::PER_THREAD];
    int q0, ks;
    __device__ __forceinline__ void init(int k_begin)
    {
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(src), 0, (int)((int64_t)nrb * ksteps * 1024), 0x00020000);
        ks = (int)threadIdx.x >> 6;
        q0 = (k_begin >> 4) + ks;
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p)
            off[p] = (rb0 + p < nrb) ? ((uint32_t)(rb0 + p) * (uint32_t)ksteps + (uint32_t)q0) * 1024u + ((uint32_t)threadIdx.x & 63u) * 16u
                                     : BUFFER_OOB;
    }
    __device__ __forceinline__ void load_piece(f32x4 &reg, int p, int stage) const
    {
        const uint32_t adv = (q0 + stage * Tile::KS < klim_steps) ? (uint32_t)stage * (uint32_t)(Tile::KS * 1024) : BUFFER_OOB;
        reg = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(off[p] + adv), 0, 0));
    }
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int stage) const
    {
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p) load_piece(regs[p], p, stage);
    }
};

// A value the optimiser cannot trace back to threadIdx.x: addresses computed from it inside the tile loop stay inside the
// loop instead of being computed once, kept in registers over the main loop and spilled.
__device__ __forceinline__ int opaque_tid()
{
    int t = (int)threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

// ----------------------------------------------------------------------------------------------- the persistent pipeline
// Registers of one operand pair: the BIG_DEPTH stages requested ahead of the one being multiplied (stage j lives in slot
// j % BIG_DEPTH).  Measured at 4096 tokens, 14336 features, k = 1024: a depth of two stages is no faster than one and leaves
// no registers for anything else.
constexpr int BIG_DEPTH = 1;
template <class PA, class PB> struct BigRegs {
    f32x4 ra[BIG_DEPTH][PA::Tile::PER_THREAD], rb[BIG_DEPTH][PB::Tile::PER_THREAD];
};

// Requests the first BIG_DEPTH stages of a tile (providers filled in by the caller).
template <class PA, class PB> __device__ __forceinline__ void big_prefetch(BigRegs<PA, PB> &r, PA &pa, PB &pb, int k_begin)
{
    pa.init(k_begin);
    pb.init(k_begin);
#pragma unroll
    for (int j = 0; j < BIG_DEPTH; ++j) {
        pa.load(r.ra[j], j);
        pb.load(r.rb[j], j);
    }
}

// One stage of 4 k-steps, entered right after the barrier that completed LDS buffer `cur`.  The last k-step of a stage is not
// multiplied inside its own stage: its fragments (fa[1], fb[1] on entry) wait in registers across the barrier and their
// MFMAs run here first, while this stage's first fragments come in from LDS.  With one wave per SIMD nothing else would cover
// that wait.  Between the MFMAs, as in pipeline_stage: the registers ra / rb (a later stage) go to the idle buffer `oth` and
// are refilled with stages next_a / next_b.
template <int MI, int NI, class PA, class PB>
__device__ __forceinline__ void big_stage(f32x16 (&acc)[MI][NI], const bf16_t *__restrict__ cur, bf16_t *__restrict__ oth,
                                          f32x4 (&ra)[PA::Tile::PER_THREAD], f32x4 (&rb)[PB::Tile::PER_THREAD], const PA &pa, const PB &pb, int next_a,
                                          int next_b, bf16x8 (&fa)[2][MI], bf16x8 (&fb)[2][NI], int arow, int brow, int lane)
{
    typedef typename PA::Tile TA;
    typedef typename PB::Tile TB;
    constexpr int KS = 4;
    constexpr int FRAG_OPS = (MI * (TA::LAYOUT_ID == M_CONT ? 2 : 1)) + (NI * (TB::LAYOUT_ID == M_CONT ? 2 : 1));
    constexpr int COPY_OPS = 2 * ((TA::PER_THREAD + TB::PER_THREAD + KS - 1) / KS);
    constexpr int MEM_PER_MFMA = (FRAG_OPS + COPY_OPS + MI * NI - 1) / (MI * NI);
    const bf16_t *As = cur, *Bs = cur + TA::LDS_ELEMS;
    // group g = 0: the pending k-step (fragments in slot 1), reads k-step 0 into slot 0; group g = 1..3: k-step g - 1 from slot
    // (g - 1) % 2, reads k-step g into slot g % 2.  k-step 3 is left in slot 1 for the next stage.
#pragma unroll
    for (int g = 0; g < KS; ++g) {
        const int use = (g + 1) & 1, fill = g & 1;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            fa[fill][mi] = TA::frag(As, arow + mi * 32, g, lane);
        }
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) fb[fill][ni] = TB::frag(Bs, brow + ni * 32, g, lane);
#pragma unroll
        for (int p = 0; p < TA::PER_THREAD; ++p)
            if (p % KS == g) {
                TA::store_piece(oth, ra[p], p);
                pa.load_piece(ra[p], p, next_a);
            }
#pragma unroll
        for (int p = 0; p < TB::PER_THREAD; ++p)
            if ((p + TA::PER_THREAD) % KS == g) {
                TB::store_piece(oth + TA::LDS_ELEMS, rb[p], p);
                pb.load_piece(rb[p], p, next_b);
            }
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[use][mi], fb[use][ni], acc[mi][ni], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < MI * NI; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x090, MEM_PER_MFMA, 0);  // then vector-memory / LDS instructions
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
}

// Contracts `nstage` stages of 64 into acc; the first stages are in r (big_prefetch).  `lds` holds two stages and is free again
// on return (the loop ends with a barrier).  Waves as 2 x 2: a wave owns (BM / 2) x (BN / 2) of the tile.
template <int BM, int BN, class PA, class PB>
__device__ __forceinline__ void big_mainloop(f32x16 (&acc)[BM / 64][BN / 64], bf16_t *__restrict__ lds, BigRegs<PA, PB> &r, PA &pa, PB &pb, int nstage)
{
    typedef typename PA::Tile TA;
    typedef typename PB::Tile TB;
    constexpr int MI = BM / 64, NI = BN / 64, STAGE = TA::LDS_ELEMS + TB::LDS_ELEMS;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, arow = (wave >> 1) * MI * 32, brow = (wave & 1) * NI * 32;
    TA::store(lds, r.ra[0]);
    TB::store(lds + TA::LDS_ELEMS, r.rb[0]);
    pa.load(r.ra[0], BIG_DEPTH);
    pb.load(r.rb[0], BIG_DEPTH);
    // the pending k-step of the first stage: zeros
    bf16x8 fa[2][MI], fb[2][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int e = 0; e < 8; ++e) fa[1][mi][e] = (__bf16)0.0f;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int e = 0; e < 8; ++e) fb[1][ni][e] = (__bf16)0.0f;
    __syncthreads();
    // One loop body for all stages, the last ones included: what they request lies past the contraction's end and comes back as
    // zeros without touching memory, and what they hand to LDS is never read.  (With the last trip peeled off, the compiler
    // gives the 256 accumulator registers a different assignment in the peeled copy and moves them all at the loop's exit.)
    // Stage s is in LDS buffer s % 2; while it is multiplied, the slot of stage s + 1 goes to the other buffer and is refilled with
    // stage s + 1 + BIG_DEPTH.
    const int nround = (nstage + 1) / 2 * 2;
    for (int s = 0; s < nround; s += 2) {
        big_stage<MI, NI>(acc, lds, lds + STAGE, r.ra[1 % BIG_DEPTH], r.rb[1 % BIG_DEPTH], pa, pb, s + 1 + BIG_DEPTH, s + 1 + BIG_DEPTH, fa, fb, arow, brow, lane);
        big_stage<MI, NI>(acc, lds + STAGE, lds, r.ra[0], r.rb[0], pa, pb, s + 2 + BIG_DEPTH, s + 2 + BIG_DEPTH, fa, fb, arow, brow, lane);
    }
    // the last stage's last k-step
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][mi], fb[1][ni], acc[mi][ni], 0, 0, 0);
}

template <int BM, int BN> __device__ __forceinline__ void big_zero(f32x16 (&acc)[BM / 64][BN / 64])
{
#pragma unroll
    for (int mi = 0; mi < BM / 64; ++mi)
#pragma unroll
        for (int ni = 0; ni < BN / 64; ++ni) acc[mi][ni] = zero16();
}

// ----------------------------------------------------------------------------------------------- epilogues
// One accumulator value, copied out of the accumulator registers where the epilogue uses it.  Written as an instruction: left
// to itself the compiler copies all 256 accumulators into ordinary registers at the end of the main loop (the vector ALU cannot
// read accumulator registers) and spills whatever else was live.  Callers pass a few idle cycles after the last matrix
// instruction first (acc_settle), since the hardware's wait for a matrix result is not inserted around inline instructions.
__device__ __forceinline__ float acc_read(float a)
{
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}
template <int MI, int NI> __device__ __forceinline__ void acc_settle(f32x16 (&acc)[MI][NI])
{
    // the empty statements pin every accumulator's last MFMA before the idle cycles (instructions written out like these keep
    // their order among themselves, and these take the accumulators as operands)
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) asm volatile("" : "+a"(acc[mi][ni]));
    // 96 idle cycles: a 32 x 32 x 16 MFMA occupies the matrix core for 32 and the last of a run may have been issued just before
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15");
}

// The bias values of a thread's accumulator rows, as they lie in memory (four bf16 per accumulator quad), requested before the
// tile's main loop so that the epilogue never waits for them: zeros past na, and everywhere when there is no bias (an empty
// buffer).  bias 8-byte aligned.
template <int BM> struct BigBias {
    uint2 w[BM / 64 * 4];
};
template <int BM> __device__ __forceinline__ void big_load_bias(BigBias<BM> &bw, const bf16_t *__restrict__ bias, int a0, int na)
{
    constexpr int MI = BM / 64;
    const int t = threadIdx.x, wave = t >> 6, g = (t & 63) >> 5, wm = wave >> 1;
    static const __device__ uint32_t no_bias[2] = {0u, 0u};   // base of the empty buffer
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(bias ? (const void *)bias : (const void *)no_bias), 0, bias ? na * 2 : 0, 0x00020000);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int jq = 0; jq < 4; ++jq)
            bw.w[mi * 4 + jq] =
                __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(rs, (a0 + wm * MI * 32 + mi * 32 + 8 * jq + 4 * g) * 2, 0, 0));
}

template <int BM, int BN, bool BIAS, bool STREAM = false>
__device__ __forceinline__ void big_store_bf16(f32x16 (&acc)[BM / 64][BN / 64], bf16_t *__restrict__ lds, bf16_t *__restrict__ out, int64_t ld,
                                               int64_t out_elems, int a0, int na, int b0, int nb, const BigBias<BM> &bw, int t)
{
    constexpr int MI = BM / 64, NI = BN / 64, LDS_LD = BM + 8;
    const int wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave >> 1, wn = wave & 1;
    acc_settle<BM / 64, BN / 64>(acc);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
            const int a = wm * MI * 32 + mi * 32 + 8 * jq + 4 * g;
            float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (BIAS) {
                const uint2 q = bw.w[mi * 4 + jq];
                bv[0] = __uint_as_float(q.x << 16);
                bv[1] = __uint_as_float(q.x & 0xffff0000u);
                bv[2] = __uint_as_float(q.y << 16);
                bv[3] = __uint_as_float(q.y & 0xffff0000u);
            }
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int b = wn * NI * 32 + ni * 32 + r;
                store4<bf16_t>(lds + b * LDS_LD + a, acc_read(acc[mi][ni][jq * 4 + 0]) + bv[0], acc_read(acc[mi][ni][jq * 4 + 1]) + bv[1],
                               acc_read(acc[mi][ni][jq * 4 + 2]) + bv[2], acc_read(acc[mi][ni][jq * 4 + 3]) + bv[3]);
            }
        }
    __syncthreads();
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)(out_elems * 2), 0x00020000);
    constexpr int PIECES = BM * BN / 8 / 256, GROUP = 8;
    static_assert(PIECES % GROUP == 0, "pieces leave in groups of 8");
    const int a = (t % (BM / 8)) * 8, bq = t / (BM / 8);   // 256 % (BM / 8) == 0: a thread's pieces share their columns
    const bool a_ok = a0 + a < na;
    // eight pieces are read from LDS before the first of them is stored: one wait for LDS per group instead of one per piece
#pragma unroll
    for (int p0 = 0; p0 < PIECES; p0 += GROUP) {
        f32x4 v[GROUP];
#pragma unroll
        for (int q = 0; q < GROUP; ++q) v[q] = *reinterpret_cast<const f32x4 *>(lds + ((p0 + q) * (256 / (BM / 8)) + bq) * LDS_LD + a);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < GROUP; ++q) {
            const int b = (p0 + q) * (256 / (BM / 8)) + bq;
            const uint32_t off = (a_ok && b0 + b < nb) ? (uint32_t)(((int64_t)(b0 + b) * ld + a0 + a) * 2) : BUFFER_OOB;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v[q]), rs, (int)off, 0, STREAM ? 2 : 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
}

// D[a][b] as fp32 to out[(a0 + a) * ld + b0 + b]: each wave passes its quadrant through an LDS patch of 32 rows x its
// BN / 2 columns (row stride + 4 floats), so that a lane stores 16 bytes of a row.  Pieces outside na x nb are dropped by the
// buffer bounds check.  `out` holds out_elems < 2^29 floats; nb, ld multiples of 4.  Non-temporal: the sums are for a later launch.
constexpr uint32_t BUFFER_OOB_ANY = 0xfffffff0u;   // outside a buffer of any size up to 2^32 - 16 bytes
template <int BM, int BN>
__device__ __forceinline__ void big_store_f32(f32x16 (&acc)[BM / 64][BN / 64], bf16_t *__restrict__ lds, float *__restrict__ out, int64_t ld,
                                              int64_t out_elems, int a0, int na, int b0, int nb, int t)
{
    constexpr int MI = BM / 64, NI = BN / 64, COLS = NI * 32, LDP = COLS + 4;
    const int wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave >> 1, wn = wave & 1;
    float *patch = reinterpret_cast<float *>(lds) + wave * 32 * LDP;
    acc_settle<BM / 64, BN / 64>(acc);
    constexpr int LPR = COLS / 4;                 // lanes per row of the patch
    constexpr int RPP = 64 / LPR;                 // rows per pass
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)(out_elems * 4), 0x00020000);
    const int col = (lane % LPR) * 4, b = b0 + wn * COLS + col;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int j = 0; j < 16; ++j) patch[(8 * (j / 4) + 4 * g + (j % 4)) * LDP + ni * 32 + r] = acc_read(acc[mi][ni][j]);
        __builtin_amdgcn_sched_barrier(0);   // a quarter of the accumulators at a time (see big_store_bf16)
        __builtin_amdgcn_wave_barrier();   // LDS serves a wave's instructions in order: the reads see these writes
#pragma unroll
        for (int q = 0; q < 32 / RPP; ++q) {
            const int row = q * RPP + lane / LPR;
            const int a = a0 + wm * MI * 32 + mi * 32 + row;
            const uint32_t off = (a < na && b < nb) ? (uint32_t)(((int64_t)a * ld + b) * 4) : BUFFER_OOB_ANY;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, *reinterpret_cast<const f32x4 *>(patch + row * LDP + col)), rs, (int)off, 0, 2);
        }
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();   // the patches lie where the next tile's first stage goes
}

// Dynamic LDS of a kernel on this engine: two stages of both operands, or the bf16 output tile, or the fp32 patches.
template <int BM, int BN, class TA, class TB> constexpr size_t big_smem()
{
    constexpr size_t stages = 2 * (size_t)(TA::LDS_ELEMS + TB::LDS_ELEMS) * sizeof(bf16_t);
    constexpr size_t store16 = (size_t)BN * (BM + 8) * sizeof(bf16_t);
    constexpr size_t store32 = (size_t)4 * 32 * (BN / 2 + 4) * sizeof(float);
    return stages > store16 ? (stages > store32 ? stages : store32) : (store16 > store32 ? store16 : store32);
}

// Item `idx` of a cost-sorted list goes to the blocks in rows that run alternately forwards and backwards, so that the blocks
// that got the most expensive items of one row get the cheapest of the next.  Item of block b in round r:
__device__ __forceinline__ int big_item(int b, int r, int nblocks) { return r * nblocks + ((r & 1) ? nblocks - 1 - b : b); }

}  // namespace rdb
