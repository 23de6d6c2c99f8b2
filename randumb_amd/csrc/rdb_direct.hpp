// Tile engine variant in which one operand never passes through LDS.
//
// The two long contractions of the backward pass, t = dy . C and dC = dy^T . z, each multiply the big activation gradient dy
// with a small matrix (C: out_f x k, z: tokens x k) that every block re-reads.  When the small matrix lies in memory in MFMA
// fragment order, a wave fetches its fragments with one coalesced 1 KB load per k-step straight into registers: no
// register->LDS copy, no fragment read, no bank conflicts for that operand, and LDS holds only the dy tile.
//
// The producers of the fragment-ordered copies are factored_z_kernel (z transposed, and C transposed, beside z itself);
// the layout of the buffer they live in ("projection state") is ProjLayout below.
#pragma once
#include "rdb_gemm.hpp"

namespace rdb {

// ----------------------------------------------------------------------------------------------- fragment order
// A matrix M[row][kk] in fragment order, rows padded to 32 and kk to 16: k-step s of row block j is 1 KB,
//   element (row, kk) -> ((row / 32) * ksteps + kk / 16) * 512 + ((kk / 8) % 2 * 32 + row % 32) * 8 + kk % 8,
// i.e. lane (row % 32, (kk / 8) % 2) of a wave holds 8 consecutive kk: the register image of one MFMA operand.
__host__ __device__ inline int64_t frag_index(int64_t row, int64_t kk, int64_t ksteps)
{
    return ((row >> 5) * ksteps + (kk >> 4)) * 512 + ((((kk >> 3) & 1) << 5) + (row & 31)) * 8 + (kk & 7);
}

// Where the pieces of a layer's projection state lie in the caller's buffer (a pure function of the layer's sizes).
//   header : 256 bytes; word 0 = 1 when the transposed coefficients below are present; word 1 != 0: a launch that waits for its
//            own earlier blocks gave up waiting (never seen; the results of that launch are then undefined)
//   zf     : z = x . N^T for the forward product: fragment order [tokens32 / 32][kpad / 16], rows = tokens
//   ztf    : z transposed, fragment order, rows = coefficients: [kpad / 32][tokens64 / 16]   (operand of dC = dy^T . z)
//   ctf    : C transposed, fragment order, rows = coefficients: [kpad / 32][out64 / 16]      (operand of t = dy . C)
//   sync   : per 256 tokens, one 64-bit slot per projection tile (32 coefficients) with the tag of the launch that wrote the tile
//            last, and one counter of the blocks that have consumed them: for the forward launch whose later blocks consume
//            what its earlier blocks project
// kpad, tokens64, out64: rounded up to 64; tokens32: to 32.
struct ProjLayout {
    bool ok, fits_regs;   // fits_regs: k <= 256, the forward product keeps a token's whole contraction in registers
    int kpad;
    int64_t tok32, tok64, out64;
    int64_t zf_off, ztf_off, ctf_off, sync_off, bytes;
};

constexpr int PROJ_FRAG_KMAX = 256;   // the forward kernel that takes z in fragment order keeps k <= 256 in registers

inline ProjLayout proj_layout(const rdb_linear_desc *d)
{
    ProjLayout L = {};
    if (d->act_dtype != RDB_BF16 || d->coef_rows == 0 || d->k % 8 || d->in_f % 8 || d->out_f % 8 || d->k <= 0 || d->tokens <= 0 ||
        d->in_f <= 0 || d->out_f <= 0)
        return L;
    L.kpad = (int)(cdiv(d->k, 64) * 64);
    L.tok32 = cdiv(d->tokens, 32) * 32;
    L.tok64 = cdiv(d->tokens, 64) * 64;
    L.out64 = cdiv(d->out_f, 64) * 64;
    // every piece is addressed with 32-bit byte offsets through a buffer descriptor
    if (L.tok64 * L.kpad >= (1ll << 29) || L.out64 * L.kpad >= (1ll << 29) || d->tokens * d->k >= (1ll << 29) || d->out_f * d->k >= (1ll << 29))
        return L;
    L.fits_regs = d->k <= PROJ_FRAG_KMAX;
    auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
    L.zf_off = 256;
    L.ztf_off = L.zf_off + up(L.tok32 * L.kpad * 2);
    L.ctf_off = L.ztf_off + up(L.tok64 * L.kpad * 2);
    L.sync_off = L.ctf_off + up(L.out64 * L.kpad * 2);
    L.bytes = L.sync_off + up(cdiv(d->tokens, 256) * (L.kpad / 32 + 1) * 8);
    L.ok = true;
    return L;
}

// ----------------------------------------------------------------------------------------------- direct operand
// Fragments of a fragment-ordered matrix, for one wave: row blocks rb0 .. rb0 + NB - 1.  Loads past the end of the matrix
// fail the buffer bounds check and return zeros; loads of k-steps past the caller's contraction range return finite values
// that meet zeros of the other operand.
struct FragSource {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t base;       // byte offset of (row block rb0, k-step 0) + this lane's 16 bytes
    uint32_t rb_stride;  // bytes from one row block to the next
    __device__ __forceinline__ void init(const bf16_t *src, int64_t total_elems, int ksteps, int rb0, int lane)
    {
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(src), 0, (int)(total_elems * 2), 0x00020000);
        rb_stride = (uint32_t)ksteps * 1024u;
        base = (uint32_t)rb0 * rb_stride + (uint32_t)lane * 16u;
    }
    __device__ __forceinline__ bf16x8 load(int j, int kstep) const
    {
        return __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(base + (uint32_t)j * rb_stride + (uint32_t)kstep * 1024u), 0, 0));
    }
};

// One stage (KS k-steps of 16) with the staged operand in LDS buffer `cur` and the direct operand's fragments in
// ring[U * KS .. U * KS + KS - 1].  Between the MFMAs: the staged operand's registers (the stage after this one) go to the idle
// buffer and are refilled with stage next_s; the ring slots just used are refilled with k-steps ring_next .. ring_next + KS - 1.
template <int SI, int DI, int KS, bool STAGED_IS_A, int U, int RING, bool STORE, bool RELOAD, class PS>
__device__ __forceinline__ void direct_stage(f32x16 (&acc)[STAGED_IS_A ? SI : DI][STAGED_IS_A ? DI : SI], const bf16_t *__restrict__ cur,
                                             bf16_t *__restrict__ oth, f32x4 (&rs)[PS::Tile::PER_THREAD], const PS &ps, int next_s,
                                             bf16x8 (&ring)[RING][DI], const FragSource &fd, int ring_next, int srow, int lane)
{
    typedef typename PS::Tile TS;
    constexpr int COPY_OPS = ((STORE ? 1 : 0) + (RELOAD ? 1 : 0)) * ((TS::PER_THREAD + KS - 1) / KS) + (RELOAD ? DI : 0) +
                             (KS > 4 ? SI * (TS::LAYOUT_ID == M_CONT ? 2 : 1) : 0);
    constexpr int MEM_PER_MFMA = (COPY_OPS + SI * DI - 1) / (SI * DI);
    // fragment reads run FA k-steps ahead of the MFMAs that use them (LDS returns them in order, each k-step waits for its own
    // only): a k-step is 64 to 128 clocks of matrix work, a fragment read takes longer than that to come back
    constexpr int FA = KS < 4 ? KS : 4;
    bf16x8 fs[KS][SI];
#pragma unroll
    for (int ks = 0; ks < FA; ++ks)
#pragma unroll
        for (int i = 0; i < SI; ++i) fs[ks][i] = TS::frag(cur, srow + i * 32, ks, lane);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        if (ks + FA < KS) {
#pragma unroll
            for (int i = 0; i < SI; ++i) fs[ks + FA][i] = TS::frag(cur, srow + i * 32, ks + FA, lane);
        }
#pragma unroll
        for (int p = 0; p < TS::PER_THREAD; ++p)
            if (p % KS == ks) {
                if (STORE) TS::store_piece(oth, rs[p], p);
                if (RELOAD) ps.load_piece(rs[p], p, next_s);
            }
#pragma unroll
        for (int i = 0; i < SI; ++i)
#pragma unroll
            for (int j = 0; j < DI; ++j) {
                if (STAGED_IS_A)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fs[ks][i], ring[U * KS + ks][j], acc[i][j], 0, 0, 0);
                else
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[U * KS + ks][j], fs[ks][i], acc[j][i], 0, 0, 0);
            }
        if (RELOAD) {
#pragma unroll
            for (int j = 0; j < DI; ++j) ring[U * KS + ks][j] = fd.load(j, ring_next + ks);
        }
#pragma unroll
        for (int i = 0; i < SI * DI; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x090, MEM_PER_MFMA, 0);  // then vector-memory / LDS instructions
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
}

// Main loop: D += S . Dm over `nstage` stages of BK = 16 KS starting at contraction index k_begin (a multiple of 16).
// S: staged operand (provider PS, rows split over WS waves, SI = rows / (32 WS) fragments per wave);
// Dm: direct operand, DI row blocks per wave, fragments of k-step q at fd.load(j, q) (absolute k-step numbers).
// TRIP (2 or 4): stages per unrolled trip; DSTG (1, 2 or 4, dividing TRIP): how many stages ahead of the LDS copy the staged
// operand's registers are loaded (it comes from HBM: a load takes several stages to return under load); RD (1 or 2, dividing
// TRIP): depth of the ring of direct fragments, in stages (they come from L2).  `lds` holds 2 * PS::Tile::LDS_ELEMS elements.
template <int SI, int DI, int KS, bool STAGED_IS_A, int TRIP, int DSTG, int RD, class PS>
__device__ __forceinline__ void direct_mainloop(f32x16 (&acc)[STAGED_IS_A ? SI : DI][STAGED_IS_A ? DI : SI], bf16_t *__restrict__ lds, PS &ps,
                                                const FragSource &fd, int k_begin, int nstage, int srow, int lane)
{
    typedef typename PS::Tile TS;
    static_assert(TRIP == 2 || TRIP == 4, "the LDS double buffer needs an even trip");
    static_assert((DSTG == 1 || DSTG == 2 || DSTG == 4) && TRIP % DSTG == 0, "prefetch depth of the staged operand");
    static_assert((RD == 1 || RD == 2) && TRIP % RD == 0, "depth of the fragment ring");
    constexpr int RING = RD * KS, STAGE = TS::LDS_ELEMS;
    if (nstage <= 0) return;
    RDB_STAMP(0);
    ps.init(k_begin);
    const int q0 = k_begin >> 4;
    bf16x8 ring[RING][DI];
    f32x4 rs[DSTG][TS::PER_THREAD];
    {
        f32x4 rs0[TS::PER_THREAD];
        ps.load(rs0, 0);
#pragma unroll
        for (int j = 1; j <= DSTG; ++j) ps.load(rs[j % DSTG], j);
#pragma unroll
        for (int q = 0; q < RING; ++q)
#pragma unroll
            for (int j = 0; j < DI; ++j) ring[q][j] = fd.load(j, q0 + q);
        TS::store(lds, rs0);
    }
    __syncthreads();
    RDB_STAMP(1);
    const int nround = (nstage + TRIP - 1) / TRIP * TRIP;
    // stage s + u: LDS buffer u % 2; register slot (u + 1) % DSTG holds stage s + u + 1 and is refilled with stage s + u + 1 + DSTG;
    // ring slots (u % RD) * KS .. hold its k-steps and are refilled with those of stage s + u + RD
#define RDB_DIRECT_STAGE(U, ST, RL, NEXT_S, NEXT_Q)                                                                                  \
    direct_stage<SI, DI, KS, STAGED_IS_A, (U) % RD, RING, ST, RL>(acc, lds + ((U) & 1) * STAGE, lds + (((U) & 1) ^ 1) * STAGE, rs[((U) + 1) % DSTG], \
                                                               ps, NEXT_S, ring, fd, NEXT_Q, srow, lane)
    int s = 0;
    for (; s + TRIP < nround; s += TRIP) {
        RDB_DIRECT_STAGE(0, true, true, s + 1 + DSTG, q0 + (s + RD) * KS);
        RDB_DIRECT_STAGE(1, true, true, s + 2 + DSTG, q0 + (s + 1 + RD) * KS);
        if (TRIP == 4) {
            RDB_DIRECT_STAGE(2, true, true, s + 3 + DSTG, q0 + (s + 2 + RD) * KS);
            RDB_DIRECT_STAGE(3, true, true, s + 4 + DSTG, q0 + (s + 3 + RD) * KS);
        }
    }
    // last trip: the staged operand has nothing more to load (everything past the end reads as zeros anyway), the ring is
    // refilled only as far as the trip itself still needs, and the last stage has nothing left to hand to LDS
    if (TRIP == 2) {
        if (RD == 2) RDB_DIRECT_STAGE(0, true, false, 0, 0);
        else RDB_DIRECT_STAGE(0, true, true, nround, q0 + (s + 1) * KS);   // the ring holds one stage: the last one is still to be fetched
        RDB_DIRECT_STAGE(1, false, false, 0, 0);
    } else {
        if (RD == TRIP) {
            RDB_DIRECT_STAGE(0, true, false, 0, 0);
            RDB_DIRECT_STAGE(1, true, false, 0, 0);
        } else {   // the ring holds stages s, s + 1 (RD = 2) or s (RD = 1): stages s + RD .. s + 3 are still to be fetched
            RDB_DIRECT_STAGE(0, true, true, nround, q0 + (s + RD) * KS);
            if (RD == 1) RDB_DIRECT_STAGE(1, true, true, nround, q0 + (s + 1 + RD) * KS);
            else RDB_DIRECT_STAGE(1, true, true, nround, q0 + (s + 1 + RD) * KS);
        }
        if (RD == 1) RDB_DIRECT_STAGE(2, true, true, nround, q0 + (s + 2 + RD) * KS);
        else RDB_DIRECT_STAGE(2, true, false, 0, 0);
        RDB_DIRECT_STAGE(3, false, false, 0, 0);
    }
#undef RDB_DIRECT_STAGE
    RDB_STAMP(2);
}

}  // namespace rdb
