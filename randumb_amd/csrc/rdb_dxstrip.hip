// Input gradient of the fused linear layer, matrix-coef + bf16, for the algorithm that does form the weight:
//
//   dx[t, i] = sum_o dy[t, o] * W[o, i],   W[o, i] = sum_m C[o, m] * noise(PRIME*i + m)
//
// A block owns 128 input features x 256 tokens.  The noise columns of its features, N[i, 0:k] (they do not depend on o),
// are hashed once into LDS; then for every chunk of 64 output rows the block regenerates the weight chunk W[chunk, i] on
// the matrix cores (C chunk x noise strip, fp32 accumulation, one rounding to bf16 as materialize().to(bf16) does,
// src/rten_cpp/RandumbTensor.py:892) into LDS and multiplies the dy tile with it.  W never leaves the chip; with 256 tokens
// per block the regeneration costs as many MFMAs as the product itself.
// Replaces autograd's MmBackward on the re-materialised weight (RandumbTensor.py:942-946).
#include "rdb_gemm.hpp"
#include "rdb_tile.hpp"

namespace rdb {

constexpr int XS_BI = 128, XS_BT = 256, XS_BO = 64, XS_KMAX = 256;
constexpr int XS_LDW = XS_BO + 8;  // row stride (elements) of the W chunk and dy tiles: 144 bytes, conflict-free fragment reads

struct DxStripParams {
    const bf16_t *dy;
    const bf16_t *coef;
    bf16_t *dx;
    int64_t lddy, lddx;
    int tokens, in_f, out_f, k;
    int tiles_i, tiles_t;
    uint32_t seed;
};

// KG = k rounded up to groups of 64 coefficients (compile time, so that the regeneration is one straight line of code).
template <int KG> __global__ __launch_bounds__(256, 1) void linear_dx_nstrip_kernel(DxStripParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t *lds = reinterpret_cast<bf16_t *>(smem_raw);
    constexpr int kpad = KG * 64, ldk = kpad + 8;  // row stride of the noise strip and the C chunk: (64n + 8) elements
    bf16_t *Ns = lds;                         // [128 i][ldk]   2^31 * noise(i, m)
    bf16_t *Cs = Ns + XS_BI * ldk;            // [64 o][ldk]    C[o, m]
    bf16_t *Ws = Cs + XS_BO * ldk;            // [128 i][72]    W[o, i] of the chunk, transposed
    bf16_t *Ds = Ws + XS_BI * XS_LDW;         // [256 tok][72]  dy[tok, o] of the chunk
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5;
    // work item = (token tile, feature tile), feature tile fastest: neighbours share the dy stream
    const int w = xcd_work_item(blockIdx.x, p.tiles_i * p.tiles_t);
    if (w >= p.tiles_i * p.tiles_t) return;
    const int i0 = (w % p.tiles_i) * XS_BI, tok0 = (w / p.tiles_i) * XS_BT;

    const __amdgpu_buffer_rsrc_t rs_dy =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.dy), 0, (int)(((int64_t)(p.tokens - 1) * p.lddy + p.out_f) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_c =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t *>(p.coef), 0, (int)((int64_t)p.out_f * p.k * 2), 0x00020000);

    // pieces (16 bytes) of a chunk this thread copies: 8 of the dy tile, up to 8 of the C chunk
    constexpr int cpr = kpad / 8;             // pieces per C row
    constexpr int ncp = XS_BO * cpr;          // pieces of a C chunk (<= 2048)
    uint32_t off_dy[8], off_c[8];
    int c_row[8], c_lds[8];  // row of the C chunk a piece belongs to (beyond the chunk: never loaded), where it goes in Cs
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int idx = q * 256 + t;
        const int row = idx >> 3, c8 = idx & 7;
        off_dy[q] = (tok0 + row < p.tokens) ? (uint32_t)(((int64_t)(tok0 + row) * p.lddy + c8 * 8) * 2) : BUFFER_OOB;
        const int co = idx / cpr, cm = (idx % cpr) * 8;
        off_c[q] = (idx < ncp && cm < p.k) ? (uint32_t)((co * p.k + cm) * 2) : BUFFER_OOB;
        c_row[q] = idx < ncp ? co : 0x7fffffff;
        c_lds[q] = co * ldk + cm;
    }
    f32x4 rdy[8], rc[8];
    auto issue = [&](int o0) {   // global -> registers for the chunk starting at output row o0 (rows past out_f read as zeros)
        const int left = p.out_f - o0;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int idx = q * 256 + t;
            const uint32_t a = ((idx & 7) * 8 < left) ? off_dy[q] + (uint32_t)(o0 * 2) : BUFFER_OOB;
            rdy[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_dy, (int)a, 0, 0));
            const uint32_t b = (c_row[q] < left) ? off_c[q] + (uint32_t)(o0 * p.k * 2) : BUFFER_OOB;
            rc[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_c, (int)b, 0, 0));
        }
    };
    issue(0);

    // noise strip: N[i0 + row, m] for m < k, zeros up to kpad
    for (int e = t; e < XS_BI * cpr; e += 256) {
        const int row = e / cpr, m0 = (e % cpr) * 8;
        const uint32_t first = sq5_first((uint32_t)(i0 + row), (uint32_t)m0, p.seed);
        Frag8 f;
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const float lo = (m0 + 2 * h < p.k) ? (float)(int32_t)sq5_tail(first + (uint32_t)(2 * h) * SQ5_N1) : 0.0f;
            const float hi = (m0 + 2 * h + 1 < p.k) ? (float)(int32_t)sq5_tail(first + (uint32_t)(2 * h + 1) * SQ5_N1) : 0.0f;
            f.u[h] = f32x2_to_bf16x2(lo, hi);
        }
        *reinterpret_cast<f32x4 *>(Ns + row * ldk + m0) = f.f4;
    }

    // main product: D[a = i][b = tok]; waves 2 x 2, a wave owns 64 features x 128 tokens
    const int wi = wave >> 1, wt = wave & 1;
    f32x16 acc[2][4];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) acc[mi][ni] = zero16();
    // regeneration: D[a = o][b = i]; a wave owns 32 output rows x 64 features
    const int go = wave >> 1, gi = wave & 1;

    for (int o0 = 0; o0 < p.out_f; o0 += XS_BO) {
        // registers -> LDS (the previous chunk's readers passed the barrier at the end of the loop body)
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int idx = q * 256 + t;
            *reinterpret_cast<f32x4 *>(Ds + (idx >> 3) * XS_LDW + (idx & 7) * 8) = rdy[q];
            if (c_row[q] < XS_BO) *reinterpret_cast<f32x4 *>(Cs + c_lds[q]) = rc[q];
        }
        if (o0 + XS_BO < p.out_f) issue(o0 + XS_BO);  // next chunk's loads fly under this chunk's matrix work
        __syncthreads();

        // W chunk, transposed: Ws[i][o] = bf16(2^-31 * sum_m C[o, m] * (2^31 noise(i, m)))
        f32x16 wacc[2];
        wacc[0] = zero16();
        wacc[1] = zero16();
        {   // groups of 64 coefficients; a group's fragments are read while the group before it is in the matrix cores
            // (the scheduling barriers keep the compiler from sinking every read down to the MFMA that uses it)
            const bf16_t *pa = Cs + (go * 32 + r) * ldk + g * 8, *pb = Ns + (gi * 64 + r) * ldk + g * 8;
            bf16x8 fa[2][4], fb[2][4][2];
            auto rd = [&](int grp) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    fa[grp & 1][ks] = *reinterpret_cast<const bf16x8 *>(pa + grp * 64 + ks * 16);
                    fb[grp & 1][ks][0] = *reinterpret_cast<const bf16x8 *>(pb + grp * 64 + ks * 16);
                    fb[grp & 1][ks][1] = *reinterpret_cast<const bf16x8 *>(pb + 32 * ldk + grp * 64 + ks * 16);
                }
            };
            rd(0);
#pragma unroll
            for (int grp = 0; grp < KG; ++grp) {
                if (grp + 1 < KG) rd(grp + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    wacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[grp & 1][ks], fb[grp & 1][ks][0], wacc[0], 0, 0, 0);
                    wacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[grp & 1][ks], fb[grp & 1][ks][1], wacc[1], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                constexpr float S = 4.656612873077392578125e-10f;
                store4<bf16_t>(Ws + (gi * 64 + ni * 32 + r) * XS_LDW + go * 32 + 8 * jq + 4 * g, wacc[ni][jq * 4] * S, wacc[ni][jq * 4 + 1] * S,
                               wacc[ni][jq * 4 + 2] * S, wacc[ni][jq * 4 + 3] * S);
            }
        __syncthreads();
        {   // all fragments of the chunk first, then the 32 MFMAs
            bf16x8 fa[XS_BO / 16][2], fb[XS_BO / 16][4];
#pragma unroll
            for (int ks = 0; ks < XS_BO / 16; ++ks) {
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
                    fa[ks][mi] = *reinterpret_cast<const bf16x8 *>(Ws + (wi * 64 + mi * 32 + r) * XS_LDW + ks * 16 + g * 8);
#pragma unroll
                for (int ni = 0; ni < 4; ++ni)
                    fb[ks][ni] = *reinterpret_cast<const bf16x8 *>(Ds + (wt * 128 + ni * 32 + r) * XS_LDW + ks * 16 + g * 8);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < XS_BO / 16; ++ks)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 4; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][mi], fb[ks][ni], acc[mi][ni], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    }
    store_tile_bf16<XS_BI, XS_BT>(acc, lds, p.dx, p.lddx, i0, p.in_f, tok0, p.tokens, 1.0f, nullptr);
}

// Returns RDB_E_UNSUPPORTED (without setting an error) when the request does not fit this kernel.
int linear_dx_nstrip(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                     hipStream_t s)
{
    if (d->act_dtype != RDB_BF16 || d->coef_dtype != RDB_BF16 || d->coef_rows == 0 || scale_bias) return RDB_E_UNSUPPORTED;
    if (d->k < 1 || d->k > XS_KMAX || d->k % 8 || d->in_f % 8 || d->out_f % 8 || d->tokens < 1 || d->in_f < 1 || d->out_f < 1)
        return RDB_E_UNSUPPORTED;
    if (lddy % 8 || lddx % 8 || ((uintptr_t)dy & 15) || ((uintptr_t)coef & 15) || ((uintptr_t)dx & 15)) return RDB_E_UNSUPPORTED;
    if (d->tokens * lddy >= (1ll << 29) || d->out_f * d->k >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    DxStripParams p;
    p.dy = (const bf16_t *)dy;
    p.coef = (const bf16_t *)coef;
    p.dx = (bf16_t *)dx;
    p.lddy = lddy;
    p.lddx = lddx;
    p.tokens = (int)d->tokens;
    p.in_f = (int)d->in_f;
    p.out_f = (int)d->out_f;
    p.k = (int)d->k;
    p.tiles_i = (int)cdiv(d->in_f, XS_BI);
    p.tiles_t = (int)cdiv(d->tokens, XS_BT);
    p.seed = d->seed;
    const int kg = (int)cdiv(d->k, 64);
    const size_t ldk = kg * 64 + 8;
    size_t smem = ((XS_BI + XS_BO) * ldk + (size_t)(XS_BI + XS_BT) * XS_LDW) * sizeof(bf16_t);
    const size_t store = (size_t)XS_BT * (XS_BI + 8) * sizeof(bf16_t);
    if (smem < store) smem = store;
    const int items = p.tiles_i * p.tiles_t;
    switch (kg) {
    case 1: return launch_engine(linear_dx_nstrip_kernel<1>, p, items, smem, s, "linear_dx_nstrip_kernel<1>");
    case 2: return launch_engine(linear_dx_nstrip_kernel<2>, p, items, smem, s, "linear_dx_nstrip_kernel<2>");
    case 3: return launch_engine(linear_dx_nstrip_kernel<3>, p, items, smem, s, "linear_dx_nstrip_kernel<3>");
    default: return launch_engine(linear_dx_nstrip_kernel<4>, p, items, smem, s, "linear_dx_nstrip_kernel<4>");
    }
}

}  // namespace rdb
