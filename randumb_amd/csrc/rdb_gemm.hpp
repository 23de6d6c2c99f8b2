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
// Pipeline: global loads run two stages ahead in registers, one stage ahead in LDS (double buffer), one barrier per stage.
#pragma once

#include "rdb_common.hpp"

namespace rdb {

typedef short s16x4 __attribute__((ext_vector_type(4)));

enum OperandLayout { K_CONT = 0, M_CONT = 1 };

union Frag8 {
    bf16x8 v;
    s16x4 h[2];
    uint32_t u[4];
    f32x4 f4;
};

// One operand of the tile engine.  ROWS = tile rows (BM or BN), BK = contraction depth per stage.
template <int ROWS, int BK, int LAYOUT> struct OperandTile {
    static constexpr int PAD = 8;
    static constexpr int LD = (LAYOUT == K_CONT) ? (BK + PAD) : (ROWS + PAD);     // LDS row stride, elements
    static constexpr int LDS_ELEMS = (LAYOUT == K_CONT) ? ROWS * LD : BK * LD;    // per stage
    static constexpr int PIECES = ROWS * BK / 8;                                   // 16-byte pieces per stage
    static constexpr int PER_THREAD = (PIECES + 255) / 256;
    static_assert(PIECES % 256 == 0, "operand stage must split evenly over 256 threads");

    // Global -> registers.  row0: first tile row; nrows: rows of the matrix; k0: first k of the stage; nk: k extent.
    // Pieces outside the matrix read a valid address and are zeroed (rows % 8 == 0 / k % 8 == 0 is guaranteed by the host
    // for the contiguous axis, so a 16-byte piece is entirely inside or outside).
    __device__ static __forceinline__ void load(f32x4 (&regs)[PER_THREAD], const bf16_t *__restrict__ src, int64_t ld, int row0,
                                                int nrows, int k0, int nk)
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int idx = p * 256 + t;
            int row, k;
            bool ok;
            if (LAYOUT == K_CONT) {
                row = row0 + idx / (BK / 8);
                k = k0 + (idx % (BK / 8)) * 8;
            } else {
                k = k0 + idx / (ROWS / 8);
                row = row0 + (idx % (ROWS / 8)) * 8;
            }
            ok = row < nrows && k < nk;
            const int rr = ok ? row : 0, kk = ok ? k : 0;
            const bf16_t *ptr = (LAYOUT == K_CONT) ? src + (int64_t)rr * ld + kk : src + (int64_t)kk * ld + rr;
            f32x4 v = *reinterpret_cast<const f32x4 *>(ptr);
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            regs[p] = ok ? v : z;
        }
    }

    // Registers -> LDS stage.
    __device__ static __forceinline__ void store(bf16_t *__restrict__ lds, const f32x4 (&regs)[PER_THREAD])
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int idx = p * 256 + t;
            int off;
            if (LAYOUT == K_CONT)
                off = (idx / (BK / 8)) * LD + (idx % (BK / 8)) * 8;
            else
                off = (idx / (ROWS / 8)) * LD + (idx % (ROWS / 8)) * 8;
            *reinterpret_cast<f32x4 *>(lds + off) = regs[p];
        }
    }

    // Fragment of the 32-row block starting at tile row `rb` for k-step ks (16 wide) of the stage:
    // lane (r = lane % 32, g = lane / 32) gets k = ks*16 + g*8 .. +7 of row rb + r.
    __device__ static __forceinline__ bf16x8 frag(const bf16_t *__restrict__ lds, int rb, int ks, int lane)
    {
        Frag8 f;
        const int r = lane & 31, g = lane >> 5;
        if (LAYOUT == K_CONT) {
            f.v = *reinterpret_cast<const bf16x8 *>(lds + (rb + r) * LD + ks * 16 + g * 8);
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

// Accumulates one LDS stage into the wave's (MI x NI) 32x32 blocks.
template <class TA, class TB, int BK, int MI, int NI>
__device__ __forceinline__ void mma_stage(f32x16 (&acc)[MI][NI], const bf16_t *__restrict__ As, const bf16_t *__restrict__ Bs, int wm,
                                          int wn, int lane)
{
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 fa[MI], fb[NI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) fa[mi] = TA::frag(As, wm * MI * 32 + mi * 32, ks, lane);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) fb[ni] = TB::frag(Bs, wn * NI * 32 + ni * 32, ks, lane);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi], fb[ni], acc[mi][ni], 0, 0, 0);
    }
}

// ----------------------------------------------------------------------------------------------- operand providers
// A provider fills the registers of one pipeline stage: load(regs, k0) with k0 the stage's first contraction index.

// Operand read from global memory.
template <int ROWS, int BK, int LAYOUT> struct GlobalOperand {
    typedef OperandTile<ROWS, BK, LAYOUT> Tile;
    const bf16_t *src;
    int64_t ld;
    int row0, nrows, klim;  // klim: first contraction index that must read as zero
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int k0) const { Tile::load(regs, src, ld, row0, nrows, k0, klim); }
};

// Operand generated by the noise hash, tile rows = noise rows (tensor element index), contraction = coefficient index:
// element (row, k) = 2^31 * noise(PRIME*(row0 + row) + k) as bf16 (callers fold the 2^-31 into their epilogue).
template <int ROWS, int BK> struct NoiseOperandRowsAreElements {
    typedef OperandTile<ROWS, BK, K_CONT> Tile;
    int row0;
    uint32_t seed;
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int k0) const
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p) {
            const int idx = p * 256 + t;
            const int row = row0 + idx / (BK / 8), k = k0 + (idx % (BK / 8)) * 8;
            const uint32_t first = (uint32_t)row * PN1 + (uint32_t)k * SQ5_N1 + seed;
            uint32_t b[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * SQ5_N1);
            Frag8 f;
#pragma unroll
            for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
            regs[p] = f.f4;
        }
    }
};

// Same noise, tile rows = coefficient index, contraction = element index: element (row, k) = 2^31 * noise(PRIME*k + row0 + row).
template <int ROWS, int BK> struct NoiseOperandRowsAreCoefs {
    typedef OperandTile<ROWS, BK, K_CONT> Tile;
    int row0;
    uint32_t seed;
    __device__ __forceinline__ void load(f32x4 (&regs)[Tile::PER_THREAD], int k0) const
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < Tile::PER_THREAD; ++p) {
            const int idx = p * 256 + t;
            const int row = row0 + idx / (BK / 8), k = k0 + (idx % (BK / 8)) * 8;
            const uint32_t first = (uint32_t)k * PN1 + (uint32_t)row * SQ5_N1 + seed;
            uint32_t b[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = sq5_tail(first + (uint32_t)e * PN1);
            Frag8 f;
#pragma unroll
            for (int e = 0; e < 4; ++e) f.u[e] = f32x2_to_bf16x2((float)(int32_t)b[2 * e], (float)(int32_t)b[2 * e + 1]);
            regs[p] = f.f4;
        }
    }
};

// Main loop of the tile engine over `nstage` stages of BK starting at contraction index k_begin.
// `lds` must hold 2 * (PA::Tile::LDS_ELEMS + PB::Tile::LDS_ELEMS) elements.  On return every wave has passed a barrier
// after its last LDS read, so the caller may reuse `lds` at once.
template <int BM, int BN, int BK, class PA, class PB>
__device__ __forceinline__ void gemm_mainloop(f32x16 (&acc)[BM / 64][BN / 64], bf16_t *__restrict__ lds, const PA &pa, const PB &pb,
                                              int k_begin, int nstage)
{
    typedef typename PA::Tile TA;
    typedef typename PB::Tile TB;
    constexpr int MI = BM / 64, NI = BN / 64;
    constexpr int STAGE = TA::LDS_ELEMS + TB::LDS_ELEMS;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, wm = wave >> 1, wn = wave & 1;
    if (nstage <= 0) return;

    f32x4 ra[2][TA::PER_THREAD], rb[2][TB::PER_THREAD];
    // prologue: stage 0 -> LDS buffer 0, stage 1 -> registers (slot 1)
    pa.load(ra[0], k_begin);
    pb.load(rb[0], k_begin);
    pa.load(ra[1], k_begin + BK);
    pb.load(rb[1], k_begin + BK);
    TA::store(lds, ra[0]);
    TB::store(lds + TA::LDS_ELEMS, rb[0]);
    __syncthreads();

    // steady state, two stages per trip so that register slots and LDS buffers are compile-time constants
    for (int s = 0; s < nstage; s += 2) {
        // --- even stage s: compute buffer 0; register slot 1 holds stage s+1; fetch stage s+2 into slot 0
        __builtin_amdgcn_sched_barrier(0);
        pa.load(ra[0], k_begin + (s + 2) * BK);
        pb.load(rb[0], k_begin + (s + 2) * BK);
        __builtin_amdgcn_sched_barrier(0);
        mma_stage<TA, TB, BK, MI, NI>(acc, lds, lds + TA::LDS_ELEMS, wm, wn, lane);
        __builtin_amdgcn_sched_barrier(0);
        TA::store(lds + STAGE, ra[1]);
        TB::store(lds + STAGE + TA::LDS_ELEMS, rb[1]);
        __syncthreads();
        if (s + 1 >= nstage) break;
        // --- odd stage s+1: compute buffer 1; slot 0 holds stage s+2; fetch stage s+3 into slot 1
        __builtin_amdgcn_sched_barrier(0);
        pa.load(ra[1], k_begin + (s + 3) * BK);
        pb.load(rb[1], k_begin + (s + 3) * BK);
        __builtin_amdgcn_sched_barrier(0);
        mma_stage<TA, TB, BK, MI, NI>(acc, lds + STAGE, lds + STAGE + TA::LDS_ELEMS, wm, wn, lane);
        __builtin_amdgcn_sched_barrier(0);
        TA::store(lds, ra[0]);
        TB::store(lds + TA::LDS_ELEMS, rb[0]);
        __syncthreads();
    }
}

}  // namespace rdb
