// Fused linear layer, matrix-coef + fp32, any coefficient dimension and many tokens: the factored algorithm on the matrix
// cores at fp32 accuracy.  By default every operand value is split exactly into three bf16 parts on its way into LDS and a
// product runs as six bf16 matrix instructions (v_mfma_f32_32x32x16_bf16; see fg_split3): gfx950's bf16 matrix rate is 16 times
// its fp32 one, so six of them cost 3/8 of the eight fp32 instructions (v_mfma_f32_32x32x2_f32) they replace; the fp32
// instructions remain as the other mode of rdb_set_f32_split.
//
//   forward  z = x . N^T [T x k],  y = z . C^T (+ bias)
//   dx       t = dy . C  [T x k],  dx = t . N
//   dcoef    z as above,           dC = dy^T . z     (token ranges summed in a fixed order: bit-reproducible)
//
// N[m, i] = noise(PRIME*i + m) is hashed into the pipeline's LDS tiles and never stored; W = C . N is never formed.  All
// five products run on one kernel template that differs in where its two operands come from (a row-major matrix read along
// or across its rows, or the hash).  Operands, intermediate matrices and sums are fp32 in memory and in the accumulators.  (bf16 layers whose sizes keep them off
// the bf16 kernels, which want multiples of 8, run here too: bf16 matrices are read value by value and widened, z and t stay
// fp32, y and dx are rounded to bf16 once.)
// With scale_bias (W = C . N + s . R, R[o, i] = noise1d(o*in_f + i), full rank: src/rten_cpp/RandumbTensor.py:286-289) the
// random-bias share is one more product with R as the hashed operand, added on top:  y += s * x . R^T,  dx += s * dy . R,  and
// the gradient of s is <dy, x . R^T>, summed tile by tile in the epilogue of that product and block by block afterwards.
// Replaces materialize() + dense product (src/rten_cpp/RandumbTensor.py:942-946) and MmBackward's dW followed by
// materialize_bwd (RandumbTensor.py:979-990, 304-359) for fp32 layers beyond the few-token regime of rdb_smallk.hip.
#include "rdb_gemm.hpp"
#include <algorithm>
#include <type_traits>

namespace rdb {

constexpr int FG_BN = 128;        // B rows (output columns) per block
constexpr int FG_BK = 16;         // contraction values per stage
constexpr int FG_THREADS = 256;   // four waves, 2 x 2
constexpr uint32_t FG_OOB = 0x80000000u;   // a byte offset past the end of any matrix these kernels take (below 2^31 bytes)

// Where an operand's tile [rows x FG_BK] comes from.  In LDS every tile is [FG_BK][rows + 4]: an MFMA operand is 32
// consecutive floats of each of two contraction values.
enum FgSource {
    FG_KCONT = 0,    // src[row * ld + kk]: a row-major matrix whose rows are the tile's rows
    FG_MCONT = 1,    // src[kk * ld + row]: a row-major matrix whose rows are contraction values
    FG_NOISE_M = 2,  // 2-D noise (feature kk, coefficient row): the rows are coefficients, the contraction runs over features
    FG_NOISE_I = 3,  // 2-D noise (feature row, coefficient kk): the rows are features, the contraction runs over coefficients
    FG_NOISE_1D = 4  // 1-D noise at index row * sR + kk * sK: the random-bias matrix R, read along or across its rows
};
// What a block does with its accumulators.
enum FgEpilogue {
    FG_STORE = 0,       // out = acc
    FG_STORE_BIAS = 1,  // out = acc + bias[column]
    FG_ADD_SCALED = 2,  // out += scale[0] * acc
    FG_DOT = 3,         // dot_part[block] = sum over the tile of acc * dotm (nothing is stored to out)
    FG_STORE_RBIAS = 4  // out = acc + scale[0] * noise1d(row * nsR + column * nsK): materialising W = C . N + s . R
};

struct FgParams {
    const float *a;   // A operand's matrix (FG_KCONT / FG_MCONT)
    int64_t lda;
    const float *b;   // B operand's matrix; not used by the noise sources
    int64_t ldb;
    float *out;       // [M x N], leading dimension ldo; split s of the contraction writes out + s * split_stride
    int64_t ldo, split_stride;
    const float *bias;   // [N] or NULL
    int M, N, K;
    int kchunk;          // contraction values per split (a multiple of FG_BK); K when there is one split
    int64_t a_bytes, b_bytes;   // extent of the matrices, for the bounds check of the loads (< 2^31)
    uint32_t seed;
    int a_es, b_es;             // bytes per element of the A and B matrices: 4, or 2 (bf16; only the value-by-value kernels)
    int out_bf16;               // out, bias and dotm are bf16 (the activations' dtype)
    int scale_bf16;             // scale is bf16 (the coefficients' dtype)
    uint32_t nsR, nsK;          // FG_NOISE_1D: index steps per row and per contraction value
    const float *scale;         // FG_ADD_SCALED: one device value
    const float *dotm;          // FG_DOT: [M x N] matrix, leading dimension lddot
    int64_t lddot;
    float *dot_part;            // FG_DOT: one value per block, in block order (x fastest, then y)
};

// fp32 products on the bf16 matrix cores.  v = h + m + l exactly, each part a bf16 (the top 8 bits of what is left: truncation,
// so every difference is exact); a product a . b is then the sum of the nine products of the parts, each exact in the matrix
// core's fp32 accumulation, and the six largest of them, ah bh + ah bm + am bh + ah bl + al bh + am bm, leave out less than
// 2^-23 |a b|: an fp32 product's own rounding.  Six bf16 matrix instructions of 32 x 32 x 16 do the work of eight fp32 ones of
// 32 x 32 x 2 in 3/8 of the time.  (An infinite input becomes NaN: inf - inf.)  The parts come back as fp32 bit patterns with
// the low half zero.
__device__ __forceinline__ void fg_split3(float v, uint32_t &h, uint32_t &m, uint32_t &l)
{
    h = __float_as_uint(v) & 0xffff0000u;
    const float r1 = v - __uint_as_float(h);
    m = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(m);
    l = __float_as_uint(r2) & 0xffff0000u;
}

// One operand's way from its source into LDS: load(stage) requests / hashes the stage's values into registers, store() puts
// them into a tile.  Rows past `rows` and contraction values past `kend` are zeros.
// VEC: the matrix is read in pieces of four values (16 bytes of fp32, 8 bytes of bf16; 16-byte aligned base, leading dimension a
// multiple of 4, and the extent that runs along a piece a multiple of 4, so that a piece lies inside or outside as a whole);
// otherwise value by value.
// SPLIT: the tile goes to LDS as three bf16 planes (see fg_split3): planes of [2 halves of the stage's 16 contraction values]
// [rows][8] for the sources read along the contraction (a lane's MFMA operand is 16 consecutive bytes), of [16][rows + 32] for
// FG_MCONT (read back with the LDS transpose read).  The noise sources then give a thread consecutive contraction values.
template <int ROWS, int SRC, bool VEC, bool SPLIT = false> struct FgOperand {
    static constexpr int LD = ROWS + 4, TILE = FG_BK * LD, NV = ROWS * FG_BK / FG_THREADS / 4;   // float4 per thread and stage
    static_assert(NV >= 1, "a stage is at least one float4 per thread");
    static constexpr int LDM = ROWS + 32;                                            // FG_MCONT plane: elements per contraction value
    static constexpr int PLANE = SRC == FG_MCONT ? FG_BK * LDM : 2 * ROWS * 8;       // bf16 elements of one plane
    static constexpr int TILE_BYTES = SPLIT ? 3 * PLANE * 2 : TILE * 4;
    static constexpr int KPT = NV * 4;                                               // SPLIT, noise: consecutive contraction values per thread
    __amdgpu_buffer_rsrc_t rs;
    uint32_t off[NV];   // byte offset of the thread's pieces at stage 0
    bool ok[NV];        // ... and whether the piece's (first) row exists
    uint32_t step;      // bytes per stage
    uint32_t first;     // noise: first-round value of the thread's first element at stage 0
    int kk0, kend, k_begin, row_ok;
    int rows_left[NV];  // FG_MCONT without VEC: how many of the piece's four rows exist
    f32x4 r[NV];

    uint32_t inc;       // noise: first-round step per contraction value
    int es;             // bytes per element of the matrix (2: bf16, value by value only)
    __device__ __forceinline__ float load1(uint32_t o, bool in, int j) const
    {
        if (es == 2) {
            const unsigned short h = __builtin_amdgcn_raw_buffer_load_b16(rs, in ? (int)(o + 2 * j) : (int)FG_OOB, 0, 0);
            return bf16_to_f32(h);
        }
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, in ? (int)(o + 4 * j) : (int)FG_OOB, 0, 0));
    }
    // VEC: four consecutive elements at byte offset o (fp32: 16 bytes; bf16: 8 bytes, widened), zeros when outside
    __device__ __forceinline__ f32x4 load4(uint32_t o, bool in) const
    {
        if (es == 2) {
            const f32x2 h = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, in ? (int)o : (int)FG_OOB, 0, 0));
            const uint32_t lo = __float_as_uint(h[0]), hi = __float_as_uint(h[1]);
            return f32x4{__uint_as_float(lo << 16), __uint_as_float(lo & 0xffff0000u), __uint_as_float(hi << 16), __uint_as_float(hi & 0xffff0000u)};
        }
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, in ? (int)o : (int)FG_OOB, 0, 0));
    }
    __device__ __forceinline__ void init(const float *src, int64_t ld, int64_t bytes, int row0, int rows, int k_begin_, int kend_, uint32_t seed,
                                         uint32_t sR, uint32_t sK, int es_)
    {
        const int t = threadIdx.x;
        k_begin = k_begin_;
        kend = kend_;
        es = es_;
        if (SRC == FG_KCONT) {
            rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(src), 0, (int)bytes, 0x00020000);
            step = (uint32_t)(FG_BK * es);
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const int idx = h * FG_THREADS + t, row = idx >> 2, kq = idx & 3;
                ok[h] = row0 + row < rows;
                off[h] = ok[h] ? (uint32_t)(((int64_t)(row0 + row) * ld + k_begin + kq * 4) * es) : 0u;
            }
            kk0 = (t & 3) * 4;
        } else if (SRC == FG_MCONT) {
            rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(src), 0, (int)bytes, 0x00020000);
            step = (uint32_t)(FG_BK * ld * es);
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const int idx = h * FG_THREADS + t, kk = idx / (ROWS / 4), r4 = (idx % (ROWS / 4)) * 4;
                ok[h] = row0 + r4 < rows;
                off[h] = ok[h] ? (uint32_t)(((int64_t)(k_begin + kk) * ld + row0 + r4) * es) : 0u;
                rows_left[h] = rows - (row0 + r4);
            }
            kk0 = t / (ROWS / 4);
        } else {
            const int row = t % ROWS;
            kk0 = SPLIT ? (t / ROWS) * KPT : t / ROWS;
            row_ok = row0 + row < rows;
            if (SRC == FG_NOISE_1D) {
                first = ((uint32_t)(row0 + row) * sR + (uint32_t)(k_begin + kk0) * sK) * SQ5_N1 + seed;
                inc = sK * SQ5_N1;
            } else {
                first = SRC == FG_NOISE_M ? sq5_first((uint32_t)(k_begin + kk0), (uint32_t)(row0 + row), seed)
                                          : sq5_first((uint32_t)(row0 + row), (uint32_t)(k_begin + kk0), seed);
                inc = SRC == FG_NOISE_M ? PN1 : SQ5_N1;
            }
        }
    }
    __device__ __forceinline__ void load(int stage)
    {
        if (SRC == FG_KCONT) {
            // a thread's four values are consecutive contraction values
            const int kk = k_begin + stage * FG_BK + kk0;
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const uint32_t o = off[h] + (uint32_t)stage * step;
                if (VEC) {   // all inside or all outside
                    r[h] = load4(o, ok[h] && kk < kend);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) r[h][j] = load1(o, ok[h] && kk + j < kend, j);
                }
            }
        } else if (SRC == FG_MCONT) {
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const bool in = ok[h] && k_begin + stage * FG_BK + kk0 + h * (FG_THREADS / (ROWS / 4)) < kend;
                const uint32_t o = off[h] + (uint32_t)stage * step;
                if (VEC) {
                    r[h] = load4(o, in);
                } else {   // a thread's four values are consecutive rows: rows_left of them exist
#pragma unroll
                    for (int j = 0; j < 4; ++j) r[h][j] = load1(o, in && j < rows_left[h], j);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < NV * 4; ++j) hash_piece(stage, j);
        }
    }
    // Noise sources: element j of the thread's NV * 4 values of a stage (contraction value kk0 + j * (FG_THREADS / ROWS), one add
    // apart in the first round).  The main loop calls this between the matrix instructions of the stage before.
    static constexpr bool HASHED = SRC == FG_NOISE_M || SRC == FG_NOISE_I || SRC == FG_NOISE_1D;
    __device__ __forceinline__ void hash_piece(int stage, int j)
    {
        constexpr int KSTEP = SPLIT ? 1 : FG_THREADS / ROWS;
        const uint32_t f = first + (uint32_t)(stage * FG_BK + j * KSTEP) * inc;
        const bool in = row_ok && k_begin + stage * FG_BK + kk0 + j * KSTEP < kend;
        r[j >> 2][j & 3] = in ? sq5_unit(sq5_tail(f)) : 0.0f;
    }
    __device__ __forceinline__ void store(float *__restrict__ tile) const
    {
        const int t = threadIdx.x;
        if (SRC == FG_KCONT) {
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const int idx = h * FG_THREADS + t, row = idx >> 2, kq = idx & 3;
#pragma unroll
                for (int j = 0; j < 4; ++j) tile[(kq * 4 + j) * LD + row] = r[h][j];
            }
        } else if (SRC == FG_MCONT) {
#pragma unroll
            for (int h = 0; h < NV; ++h) {
                const int idx = h * FG_THREADS + t, kk = idx / (ROWS / 4), r4 = (idx % (ROWS / 4)) * 4;
                *reinterpret_cast<f32x4 *>(tile + kk * LD + r4) = r[h];
            }
        } else {
            constexpr int KSTEP = FG_THREADS / ROWS;
            const int row = t % ROWS;
#pragma unroll
            for (int j = 0; j < NV * 4; ++j) tile[(kk0 + j * KSTEP) * LD + row] = r[j >> 2][j & 3];
        }
    }
    // SPLIT: four of the thread's values into the planes, 8 bytes each, at element offset `at` of a plane.  Values that come from a
    // bf16 matrix are their own first part and the other two are zero: only the first plane is written (and read, see the kernel).
    __device__ __forceinline__ bool one_plane() const { return !HASHED && es == 2; }
    template <bool ONE> __device__ __forceinline__ void put4(bf16_t *__restrict__ tile, int at, const f32x4 &v) const
    {
        if (ONE) {
            *reinterpret_cast<uint2 *>(tile + at) = make_uint2((__float_as_uint(v[1]) & 0xffff0000u) | (__float_as_uint(v[0]) >> 16),
                                                               (__float_as_uint(v[3]) & 0xffff0000u) | (__float_as_uint(v[2]) >> 16));
            return;
        }
        uint32_t h[4], m[4], l[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) fg_split3(v[j], h[j], m[j], l[j]);
        *reinterpret_cast<uint2 *>(tile + at) = make_uint2(h[1] | (h[0] >> 16), h[3] | (h[2] >> 16));
        *reinterpret_cast<uint2 *>(tile + PLANE + at) = make_uint2(m[1] | (m[0] >> 16), m[3] | (m[2] >> 16));
        *reinterpret_cast<uint2 *>(tile + 2 * PLANE + at) = make_uint2(l[1] | (l[0] >> 16), l[3] | (l[2] >> 16));
    }
    template <bool ONE> __device__ __forceinline__ void store_split(bf16_t *__restrict__ tile) const
    {
        const int t = threadIdx.x;
        if (SRC == FG_KCONT) {
#pragma unroll
            for (int h = 0; h < NV; ++h) {   // contraction values 4 kq .. 4 kq + 3 of a row
                const int idx = h * FG_THREADS + t, row = idx >> 2, kq = idx & 3;
                put4<ONE>(tile, ((kq >> 1) * ROWS + row) * 8 + (kq & 1) * 4, r[h]);
            }
        } else if (SRC == FG_MCONT) {
#pragma unroll
            for (int h = 0; h < NV; ++h) {   // four consecutive rows at one contraction value
                const int idx = h * FG_THREADS + t, kk = idx / (ROWS / 4), r4 = (idx % (ROWS / 4)) * 4;
                put4<ONE>(tile, kk * LDM + r4, r[h]);
            }
        } else {
            const int row = t % ROWS;
#pragma unroll
            for (int h = 0; h < NV; ++h) {   // contraction values kk0 + 4 h .. + 3 of a row
                const int kk = kk0 + 4 * h;
                put4<ONE>(tile, ((kk >> 3) * ROWS + row) * 8 + (kk & 7), r[h]);
            }
        }
    }
    // SPLIT: the MFMA operand of the 32 rows from rb of one plane: lane (r, g) gets contraction values 8 g .. 8 g + 7 of row rb + r
    __device__ static __forceinline__ bf16x8 frag(const bf16_t *__restrict__ plane, int rb, int lane)
    {
        const int r = lane & 31, g = lane >> 5;
        if (SRC != FG_MCONT) return *reinterpret_cast<const bf16x8 *>(plane + (g * ROWS + rb + r) * 8);
        // 16-lane group q covers rows rb + 16 q .. + 15; source lane s of the group addresses contraction value 8 g + s / 4,
        // rows 4 (s % 4) .. + 3; result lane c receives the rows' column c for four contraction values
        Frag8 f;
        const int sl = lane & 15, q = (lane >> 4) & 1;
        const bf16_t *src = plane + (g * 8 + (sl >> 2)) * LDM + rb + q * 16 + (sl & 3) * 4;
        f.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(src));
        f.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(src + 4 * LDM));
        return f.v;
    }
};

// out[M x N] (+)= A . B^T over one split of the contraction.  Block: BM x 128 of the output, four waves as 2 x 2, a wave owns
// (BM / 2) x 64 in BM / 64 x 2 accumulator tiles.  Two LDS buffers, one barrier per stage: while a stage is multiplied the
// next one is on its way from memory (or being hashed) in registers.
template <int BM, int ASRC, int BSRC, int EPI, bool VEC, bool SPLIT = false, bool ANY16 = false>
__global__ __launch_bounds__(FG_THREADS, 2) void f32_gemm_kernel(FgParams p)
{
    typedef FgOperand<BM, ASRC, VEC, SPLIT> PA;
    typedef FgOperand<FG_BN, BSRC, VEC, SPLIT> PB;
    constexpr int MI = BM / 64, NI = 2, STAGE = (PA::TILE_BYTES + PB::TILE_BYTES) / 4;   // floats
    __shared__ __align__(16) float lds[2 * STAGE];
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 31, g = lane >> 5, wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.x * BM, n0 = blockIdx.y * FG_BN;   // the long extent (tokens, as a rule) on the grid's x
    const int k_begin = blockIdx.z * p.kchunk, kend = min(p.K, k_begin + p.kchunk);
    const int nstage = (kend - k_begin + FG_BK - 1) / FG_BK;
    PA pa;
    PB pb;
    pa.init(p.a, p.lda, p.a_bytes, m0, p.M, k_begin, kend, p.seed, p.nsR, p.nsK, p.a_es);
    pb.init(p.b, p.ldb, p.b_bytes, n0, p.N, k_begin, kend, p.seed, p.nsR, p.nsK, p.b_es);
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.0f;
    pa.load(0);
    pb.load(0);
    // The stage loop, once per number of planes of the two sides (known per launch, not per kernel: a side that comes from a
    // bf16 matrix has one plane), so that each copy is straight-line code between its barriers.
    auto stages = [&](auto a_one, auto b_one) __attribute__((always_inline)) {
        constexpr int AP = decltype(a_one)::value ? 1 : 3, BP = decltype(b_one)::value ? 1 : 3;
        for (int s = 0; s < nstage; ++s) {
            float *As = lds + (s & 1) * STAGE, *Bs = As + PA::TILE_BYTES / 4;
            if (SPLIT) {
                pa.template store_split<AP == 1>(reinterpret_cast<bf16_t *>(As));
                pb.template store_split<BP == 1>(reinterpret_cast<bf16_t *>(Bs));
            } else {
                pa.store(As);
                pb.store(Bs);
            }
            __syncthreads();   // also: every wave is done reading the other buffer (the stage before this one)
            const bool more = s + 1 < nstage;
            if (more) {
                if (!PA::HASHED) pa.load(s + 1);
                if (!PB::HASHED) pb.load(s + 1);
            }
            if (SPLIT) {
                // the stage is one k-step of the bf16 matrix instruction: three planes a side, six products a tile pair, the small
                // ones first (a side that comes from a bf16 matrix has one plane: three products, or one); the next stage's noise
                // values are hashed between the tile pairs
                const bf16_t *ap = reinterpret_cast<const bf16_t *>(As), *bp = reinterpret_cast<const bf16_t *>(Bs);
                {
                    bf16x8 fa[MI][AP], fb[NI][BP];
#pragma unroll
                    for (int pl = 0; pl < 3; ++pl) {
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi)
                            if (pl < AP) fa[mi][pl] = PA::frag(ap + pl * PA::PLANE, wm * (BM / 2) + mi * 32, lane);
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni)
                            if (pl < BP) fb[ni][pl] = PB::frag(bp + pl * PB::PLANE, wn * 64 + ni * 32, lane);
                    }
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) {
                            f32x16 c = acc[mi][ni];
                            if constexpr (AP == 3 && BP == 3) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][1], fb[ni][1], c, 0, 0, 0);
                            if constexpr (AP == 3) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][2], fb[ni][0], c, 0, 0, 0);
                            if constexpr (BP == 3) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][0], fb[ni][2], c, 0, 0, 0);
                            if constexpr (AP == 3) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][1], fb[ni][0], c, 0, 0, 0);
                            if constexpr (BP == 3) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][0], fb[ni][1], c, 0, 0, 0);
                            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mi][0], fb[ni][0], c, 0, 0, 0);
                            constexpr int GROUPS = MI * NI;
                            const int grp = mi * NI + ni;
                            if (PB::HASHED && more) {
                                constexpr int PER = (PB::NV * 4 + GROUPS - 1) / GROUPS;
#pragma unroll
                                for (int j = grp * PER; j < (grp + 1) * PER && j < PB::NV * 4; ++j) pb.hash_piece(s + 1, j);
                            }
                            if (PA::HASHED && more) {
                                constexpr int PER = (PA::NV * 4 + GROUPS - 1) / GROUPS;
#pragma unroll
                                for (int j = grp * PER; j < (grp + 1) * PER && j < PA::NV * 4; ++j) pa.hash_piece(s + 1, j);
                            }
                        }
                }
                continue;
            }
            const float *ap = As + g * PA::LD + wm * (BM / 2) + r, *bp = Bs + g * PB::LD + wn * 64 + r;
#pragma unroll
            for (int ks = 0; ks < FG_BK / 2; ++ks) {
                float fa[MI], fb[NI];
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) fa[mi] = ap[ks * 2 * PA::LD + mi * 32];
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) fb[ni] = bp[ks * 2 * PB::LD + ni * 32];
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[mi], fb[ni], acc[mi][ni], 0, 0, 0);
                // the next stage's noise values are hashed in the shadow of these matrix instructions, a share per k-step
                if (PB::HASHED && more) {
                    constexpr int PER = (PB::NV * 4 + FG_BK / 2 - 1) / (FG_BK / 2);
#pragma unroll
                    for (int j = ks * PER; j < (ks + 1) * PER && j < PB::NV * 4; ++j) pb.hash_piece(s + 1, j);
                }
                if (PA::HASHED && more) {
                    constexpr int PER = (PA::NV * 4 + FG_BK / 2 - 1) / (FG_BK / 2);
#pragma unroll
                    for (int j = ks * PER; j < (ks + 1) * PER && j < PA::NV * 4; ++j) pa.hash_piece(s + 1, j);
                }
            }
        }
    };
    typedef std::integral_constant<bool, true> One;
    typedef std::integral_constant<bool, false> Three;
    if (!SPLIT || !ANY16) {   // ANY16: one of the matrices is bf16 (only then is the choice compiled in)
        stages(Three{}, Three{});
    } else {
        const bool a1 = pa.one_plane(), b1 = pb.one_plane();
        if (PA::HASHED || !a1) {
            if (PB::HASHED || !b1) stages(Three{}, Three{});
            else stages(Three{}, One{});
        } else {
            if (PB::HASHED || !b1) stages(One{}, Three{});
            else stages(One{}, One{});
        }
    }
    // accumulator j of lane (r, g): row 8 (j / 4) + 4 g + j % 4 of the A side, column r of the B side
    float *out = p.out + (int64_t)blockIdx.z * p.split_stride;
    bf16_t *out16 = reinterpret_cast<bf16_t *>(p.out);   // bf16 outputs are never the ranges' partial matrices
    const bool o16 = p.out_bf16 != 0;
    const float scale = (EPI != FG_ADD_SCALED && EPI != FG_STORE_RBIAS) ? 0.0f
                        : p.scale_bf16 ? bf16_to_f32(reinterpret_cast<const bf16_t *>(p.scale)[0]) : p.scale[0];
    float dot = 0.0f;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int n = n0 + wn * 64 + ni * 32 + r;
        if (n >= p.N) continue;
        const float bv = EPI != FG_STORE_BIAS ? 0.0f : o16 ? bf16_to_f32(reinterpret_cast<const bf16_t *>(p.bias)[n]) : p.bias[n];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int m = m0 + wm * (BM / 2) + mi * 32 + 8 * (j >> 2) + 4 * g + (j & 3);
                if (m >= p.M) continue;
                const float a = acc[mi][ni][j];
                if (EPI == FG_DOT) {
                    const int64_t e = (int64_t)m * p.lddot + n;
                    dot = fmaf(a, o16 ? bf16_to_f32(reinterpret_cast<const bf16_t *>(p.dotm)[e]) : p.dotm[e], dot);
                } else {
                    const int64_t e = (int64_t)m * p.ldo + n;
                    if (EPI == FG_STORE_RBIAS) out[e] = fmaf(scale, noise1d((uint32_t)m * p.nsR + (uint32_t)n * p.nsK, p.seed), a);
                    else if (o16) out16[e] = f32_to_bf16(EPI == FG_ADD_SCALED ? fmaf(scale, a, bf16_to_f32(out16[e])) : a + bv);
                    else out[e] = EPI == FG_ADD_SCALED ? fmaf(scale, a, out[e]) : a + bv;
                }
            }
    }
    if (EPI == FG_DOT) {
        // lanes, then waves, in a fixed order
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) dot += __shfl_xor(dot, o);
        __syncthreads();   // the stage buffers are free
        if (lane == 0) lds[wave] = dot;
        __syncthreads();
        if (t == 0) p.dot_part[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    }
}

// out[0] = part[0] + part[1] + ... : one block, every thread a strided share in index order, then the shares in thread order
__global__ __launch_bounds__(256) void f32_sum_scalars_kernel(float *__restrict__ out, const float *__restrict__ part, int n)
{
    __shared__ float sh[256];
    float v = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) v += part[i];
    sh[threadIdx.x] = v;
    __syncthreads();
    for (int w = 128; w >= 1; w >>= 1) {
        if ((int)threadIdx.x < w) sh[threadIdx.x] += sh[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = sh[0];
}

// out[i] = part[0][i] + part[1][i] + ... in split order, four values per thread (n4 groups of four, then the n % 4 last values
// one thread each)
__global__ __launch_bounds__(256) void f32_sum_splits_kernel(float *__restrict__ out, const float *__restrict__ part, int64_t n, int64_t stride, int splits, int vec)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, n4 = vec ? n / 4 : 0;
    if (i < n4) {
        f32x4 v = *reinterpret_cast<const f32x4 *>(part + i * 4);
        for (int s = 1; s < splits; ++s) v += *reinterpret_cast<const f32x4 *>(part + s * stride + i * 4);
        *reinterpret_cast<f32x4 *>(out + i * 4) = v;
    } else if (n4 * 4 + (i - n4) < n) {
        const int64_t e = n4 * 4 + (i - n4);
        float v = part[e];
        for (int s = 1; s < splits; ++s) v += part[s * stride + e];
        out[e] = v;
    }
}

// ----------------------------------------------------------------------------------------------- host side
static bool fg_aligned16(const void *q) { return ((uintptr_t)q & 15) == 0; }
static int64_t up256(int64_t n) { return (n + 255) / 256 * 256; }

// The shapes these kernels take: matrix-coef fp32, matrices below 2^31 bytes.  Extents, leading dimensions and pointers that are
// multiples of 4 elements / 16 bytes get the kernels that read 16 bytes at a time, everything else the value-by-value ones.
static bool fg_ok(const rdb_linear_desc *d)
{
    const bool f32 = d->act_dtype == RDB_F32 && d->coef_dtype == RDB_F32, b16 = d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16;
    return (f32 || b16) && d->coef_rows != 0 && d->k > 0 && d->tokens > 0 && d->in_f > 0 && d->out_f > 0 &&
           d->tokens * d->k < (1ll << 29) && d->out_f * d->k < (1ll << 29) && d->in_f < (1 << 30) && d->out_f < (1 << 30);
}
static int fg_es(int dtype) { return dtype == RDB_BF16 ? 2 : 4; }
// Wanted whenever the shapes fit: what AUTO would run instead is the general kernel, which forms W tiles on the vector ALU at a
// few TFLOP/s, so the factored form on the matrix cores wins also where it is more flops than a product on a stored W.
static bool fg_wanted(const rdb_linear_desc *) { return true; }

// Tile height and number of contraction ranges of a product [M x N] over K.  Planned for two blocks per compute unit at a
// time (the hardware takes up to four).  A product with fewer tiles than that is cut into ranges of the contraction (at least
// min_range values each, at most max_ranges): each range leaves a partial matrix, added up in range order afterwards, so the
// result does not depend on which block finishes first.  128-row tiles unless even in ranges they would leave half of the
// compute units without a block; 64-row tiles then.
struct FgPlan {
    int bm, ranges;
};
static FgPlan fg_plan(int64_t M, int64_t N, int64_t K, int num_cus, int64_t min_range, int max_ranges)
{
    const int64_t slots = 2 * (int64_t)num_cus;
    const int64_t t128 = cdiv(M, 128) * cdiv(N, FG_BN), t64 = cdiv(M, 64) * cdiv(N, FG_BN);
    int64_t cap = K / min_range;
    if (cap > max_ranges) cap = max_ranges;
    if (cap < 1) cap = 1;
    auto ranges = [&](int64_t tiles) {
        int64_t r = slots / tiles;
        if (r > cap) r = cap;
        return r < 1 ? (int64_t)1 : r;
    };
    const int64_t r128 = ranges(t128), r64 = ranges(t64);
    if (t128 * r128 * 2 < slots) return {64, (int)r64};
    return {128, (int)r128};
}
// z = x . N^T and t = dy . C, [tokens x k] over K = in_f or out_f; dC = dy^T . z, [out_f x k] over the tokens
static FgPlan zt_plan(const rdb_linear_desc *d, int64_t K, int num_cus) { return fg_plan(d->tokens, d->k, K, num_cus, 128, 32); }
static FgPlan dc_plan(const rdb_linear_desc *d, int num_cus) { return fg_plan(d->out_f, d->k, d->tokens, num_cus, 256, 64); }

// scratch: z or t [tokens x k] and its partial matrices; for the coefficient gradient also one [out_f x k] matrix per token range
int64_t linear_f32_workspace(int op, const rdb_linear_desc *d, int num_cus)
{
    rdb_linear_desc dd = *d;
    if (op == RDB_OP_LINEAR_BWD_DCOEF) dd.coef_dtype = dd.act_dtype;   // reads no coefficients
    if (!fg_ok(&dd)) return 0;
    const int64_t zt = up256(d->tokens * d->k * 4);
    auto with_parts = [&](int64_t K) { const int r = zt_plan(d, K, num_cus).ranges; return zt * (r > 1 ? 1 + r : 1); };
    if (op == RDB_OP_LINEAR_FWD) return with_parts(d->in_f);
    if (op == RDB_OP_LINEAR_BWD_DX) return with_parts(d->out_f);
    if (op != RDB_OP_LINEAR_BWD_DCOEF) return 0;
    const int r = dc_plan(d, num_cus).ranges;
    // ... and, for the gradient of the random bias's scale, one value per 64 x 128 tile of [tokens x out_f]
    return with_parts(d->in_f) + (r > 1 ? (int64_t)r * up256(d->out_f * d->k * 4) : 0) + up256(cdiv(d->tokens, 64) * cdiv(d->out_f, FG_BN) * 4);
}

// 1 (default): the linear layers' products run as six bf16 matrix instructions on three-way splits of their operands
// (fg_split3); 0: as fp32 matrix instructions.  Process-wide (rdb_set_f32_split).
static int g_f32_split = 1;
int f32_split_mode() { return g_f32_split; }
int set_f32_split_mode(int mode)
{
    const int old = g_f32_split;
    g_f32_split = mode ? 1 : 0;
    return old;
}

struct FgProduct {
    const float *a;
    int64_t lda, a_elems;
    const float *b;
    int64_t ldb, b_elems;
    float *out;
    int64_t ldo;
    const float *bias;
    int64_t M, N, K;
    int bm;                 // tile height: 128 or 64
    int64_t kchunk;         // contraction values per range (a multiple of FG_BK); 0: one range
    int64_t split_stride;   // floats between the ranges' outputs
    uint32_t seed;
    // the random-bias products (FG_NOISE_1D on the B side): index steps, and what the epilogue does
    uint32_t nsR, nsK;
    const float *scale;     // out += scale[0] * product
    const float *dotm;      // or: dot_part[block] = <product tile, dotm tile>
    int64_t lddot;
    float *dot_part;
    // bytes per element of the A and B matrices (2: bf16), and whether out / bias / dotm and scale are bf16
    int a_es = 4, b_es = 4, out_bf16 = 0, scale_bf16 = 0;
    // the products as six bf16 matrix instructions on three-way splits of the operands (fg_split3); materialising stays on the
    // fp32 matrix instructions (its unit-coefficient results are compared bit for bit)
    bool split = f32_split_mode() != 0;
};

#define FG_LAUNCH(BM_, EPI_)                                                                                  \
    do {                                                                                                      \
        if (q.split && any16) {                                                                               \
            if (vec) f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, true, true, true><<<grid, FG_THREADS, 0, s>>>(p); \
            else f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, false, true, true><<<grid, FG_THREADS, 0, s>>>(p);    \
        } else if (q.split) {                                                                                 \
            if (vec) f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, true, true><<<grid, FG_THREADS, 0, s>>>(p);       \
            else f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, false, true><<<grid, FG_THREADS, 0, s>>>(p);          \
        } else if (vec) f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, true><<<grid, FG_THREADS, 0, s>>>(p);          \
        else f32_gemm_kernel<BM_, ASRC, BSRC, EPI_, false><<<grid, FG_THREADS, 0, s>>>(p);                    \
    } while (0)
template <int ASRC, int BSRC> static int fg_launch(const FgProduct &q, int num_cus, hipStream_t s, const char *name)
{
    if (q.a_elems >= (1ll << 29) || q.b_elems >= (1ll << 29) || q.M >= (1ll << 30) || q.N >= (1ll << 30) || q.K >= (1ll << 30)) return RDB_E_UNSUPPORTED;
    FgParams p = {};
    p.a = q.a;
    p.lda = q.lda;
    p.b = q.b;
    p.ldb = q.ldb;
    p.out = q.out;
    p.ldo = q.ldo;
    p.split_stride = q.split_stride;
    p.bias = q.bias;
    p.M = (int)q.M;
    p.N = (int)q.N;
    p.K = (int)q.K;
    p.kchunk = (int)(q.kchunk > 0 ? q.kchunk : cdiv(q.K, FG_BK) * FG_BK);
    p.a_bytes = q.a_elems * q.a_es;
    p.b_bytes = q.b_elems * q.b_es;
    p.a_es = q.a_es;
    p.b_es = q.b_es;
    p.out_bf16 = q.out_bf16;
    p.scale_bf16 = q.scale_bf16;
    p.seed = q.seed;
    p.nsR = q.nsR;
    p.nsK = q.nsK;
    p.scale = q.scale;
    p.dotm = q.dotm;
    p.lddot = q.lddot;
    p.dot_part = q.dot_part;
    const int splits = (int)cdiv(q.K, p.kchunk);
    // 16-byte pieces when both matrices allow them: aligned bases and leading dimensions, and the extent along a piece a multiple of 4
    // (along the rows of a matrix: the contraction; across them: the rows of the tile)
    auto vec_ok = [&](int src, const float *m, int64_t ld, int64_t rows) {
        if (src != FG_KCONT && src != FG_MCONT) return true;
        return fg_aligned16(m) && ld % 4 == 0 && (src == FG_KCONT ? q.K % 4 == 0 : rows % 4 == 0);
    };
    const bool vec = vec_ok(ASRC, q.a, q.lda, q.M) && vec_ok(BSRC, q.b, q.ldb, q.N);   // bf16 matrices: 8-byte pieces of four values
    const bool any16 = q.a_es == 2 || ((BSRC == FG_KCONT || BSRC == FG_MCONT) && q.b_es == 2);   // the A side is always a matrix
    if (cdiv(q.N, FG_BN) > 65535) return RDB_E_UNSUPPORTED;   // the grid's y
    const dim3 grid((unsigned)cdiv(q.M, q.bm), (unsigned)cdiv(q.N, FG_BN), (unsigned)splits);
    if (BSRC == FG_NOISE_1D) {   // the random-bias products: added on top of an output, or reduced against a matrix
        if (q.bm == 128) {
            if (q.dotm) FG_LAUNCH(128, FG_DOT);
            else FG_LAUNCH(128, FG_ADD_SCALED);
        } else {
            if (q.dotm) FG_LAUNCH(64, FG_DOT);
            else FG_LAUNCH(64, FG_ADD_SCALED);
        }
    } else if (q.scale) {        // materialising W with its random-bias share
        if (q.bm == 128) FG_LAUNCH(128, FG_STORE_RBIAS);
        else FG_LAUNCH(64, FG_STORE_RBIAS);
    } else if (q.bm == 128) {
        if (q.bias) FG_LAUNCH(128, FG_STORE_BIAS);
        else FG_LAUNCH(128, FG_STORE);
    } else {
        if (q.bias) FG_LAUNCH(64, FG_STORE_BIAS);
        else FG_LAUNCH(64, FG_STORE);
    }
    return check_launch(name);
}

static bool fg_ws_ok(int op, const rdb_linear_desc *d, int num_cus, const void *ws, int64_t bytes)
{
    return ws && fg_aligned16(ws) && bytes >= linear_f32_workspace(op, d, num_cus);
}

static int fg_sum(float *out, const float *part, int64_t n, int64_t stride, int splits, hipStream_t s)
{
    const int vec = fg_aligned16(out) ? 1 : 0;   // the partial matrices are 256-byte aligned
    f32_sum_splits_kernel<<<(unsigned)cdiv(vec ? n / 4 + n % 4 : n, 256), 256, 0, s>>>(out, part, n, stride, splits, vec);
    return check_launch("f32_sum_splits_kernel");
}

// A product whose dense output [M x N] (ldo = N) may be computed in `splits` ranges of the contraction: the ranges' partial
// matrices go to `part` (stride floats apart) and are added up into q.out in range order.
template <int ASRC, int BSRC> static int fg_launch_ranges(FgProduct q, FgPlan plan, float *part, int64_t stride, int num_cus, hipStream_t s, const char *name)
{
    int splits = plan.ranges;
    q.bm = plan.bm;
    const int kchunk = (int)(cdiv(cdiv(q.K, splits), FG_BK) * FG_BK);
    splits = (int)cdiv(q.K, kchunk);   // the ranges that hold something
    if (splits <= 1) {
        q.kchunk = 0;
        q.split_stride = 0;
        return fg_launch<ASRC, BSRC>(q, num_cus, s, name);
    }
    float *out = q.out;
    q.out = part;
    q.kchunk = kchunk;
    q.split_stride = stride;
    if (int rc = fg_launch<ASRC, BSRC>(q, num_cus, s, name)) return rc;
    return fg_sum(out, part, q.M * q.N, stride, splits, s);
}

// z[T x k] = src[T x in_f] . N^T; the partial matrices of its ranges go to `part` (room for max_ranges of them, up256(T k 4)
// bytes apart; NULL: right behind z, as many as the plan wants)
static int fg_project(float *z, const float *x, int64_t ldx, const rdb_linear_desc *d, int num_cus, hipStream_t s, float *part = nullptr,
                      int max_ranges = 1 << 30)
{
    FgProduct q = {x, ldx, (d->tokens - 1) * ldx + d->in_f, nullptr, 0, 0, z, d->k, nullptr, d->tokens, d->k, d->in_f, 128, 0, 0, d->seed};
    q.a_es = fg_es(d->act_dtype);
    const int64_t zt = up256(d->tokens * d->k * 4) / 4;
    FgPlan plan = zt_plan(d, d->in_f, num_cus);
    if (plan.ranges > max_ranges) plan.ranges = max_ranges < 1 ? 1 : max_ranges;
    return fg_launch_ranges<FG_KCONT, FG_NOISE_M>(q, plan, part ? part : z + zt, zt, num_cus, s, "f32_gemm_kernel (z = x . N^T)");
}

// The three entry points return RDB_E_UNSUPPORTED, without setting an error, when the request does not fit.
int linear_fwd_f32(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                   const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!fg_ok(d) || !fg_wanted(d) || !fg_ws_ok(RDB_OP_LINEAR_FWD, d, num_cus, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    if (d->tokens * ldx >= (1ll << 29) || d->tokens * ldy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    float *z = (float *)workspace;
    if (int rc = fg_project(z, (const float *)x, ldx, d, num_cus, s)) return rc;
    FgProduct q = {z, d->k, d->tokens * d->k, (const float *)coef, d->k, d->out_f * d->k, (float *)y, ldy, (const float *)bias,
                   d->tokens, d->out_f, d->k, fg_plan(d->tokens, d->out_f, d->k, num_cus, d->k, 1).bm, 0, 0, d->seed};
    const int b16 = d->act_dtype == RDB_BF16;
    q.b_es = fg_es(d->coef_dtype);
    q.out_bf16 = b16;
    if (int rc = fg_launch<FG_KCONT, FG_KCONT>(q, num_cus, s, "f32_gemm_kernel (y = z . C^T)")) return rc;
    if (!scale_bias) return RDB_OK;
    // y += s * x . R^T: the B side's rows are output features, index o * in_f + i
    FgProduct qr = {(const float *)x, ldx, (d->tokens - 1) * ldx + d->in_f, nullptr, 0, 0, (float *)y, ldy, nullptr, d->tokens, d->out_f, d->in_f,
                    fg_plan(d->tokens, d->out_f, d->in_f, num_cus, d->in_f, 1).bm, 0, 0, d->seed, (uint32_t)d->in_f, 1u, (const float *)scale_bias,
                    nullptr, 0, nullptr};
    qr.a_es = fg_es(d->act_dtype);
    qr.out_bf16 = b16;
    qr.scale_bf16 = d->coef_dtype == RDB_BF16;
    return fg_launch<FG_KCONT, FG_NOISE_1D>(qr, num_cus, s, "f32_gemm_kernel (y += s x . R^T)");
}

int linear_dx_f32(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                  int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!fg_ok(d) || !fg_wanted(d) || !fg_ws_ok(RDB_OP_LINEAR_BWD_DX, d, num_cus, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    if (d->tokens * lddx >= (1ll << 29) || d->tokens * lddy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    float *t = (float *)workspace;
    // t[T x k] = dy[T x out_f] . C: the B side's rows are coefficients, read across the rows of C
    FgProduct q1 = {(const float *)dy, lddy, (d->tokens - 1) * lddy + d->out_f, (const float *)coef, d->k, d->out_f * d->k, t, d->k, nullptr,
                    d->tokens, d->k, d->out_f, 128, 0, 0, d->seed};
    const int b16 = d->act_dtype == RDB_BF16;
    q1.a_es = fg_es(d->act_dtype);
    q1.b_es = fg_es(d->coef_dtype);
    const int64_t zt = up256(d->tokens * d->k * 4) / 4;
    if (int rc = fg_launch_ranges<FG_KCONT, FG_MCONT>(q1, zt_plan(d, d->out_f, num_cus), t + zt, zt, num_cus, s, "f32_gemm_kernel (t = dy . C)")) return rc;
    // dx[T x in_f] = t . N: the B side's rows are input features, hashed
    FgProduct q2 = {t, d->k, d->tokens * d->k, nullptr, 0, 0, (float *)dx, lddx, nullptr, d->tokens, d->in_f, d->k,
                    fg_plan(d->tokens, d->in_f, d->k, num_cus, d->k, 1).bm, 0, 0, d->seed};
    q2.out_bf16 = b16;
    if (int rc = fg_launch<FG_KCONT, FG_NOISE_I>(q2, num_cus, s, "f32_gemm_kernel (dx = t . N)")) return rc;
    if (!scale_bias) return RDB_OK;
    // dx += s * dy . R: the B side's rows are input features, index o * in_f + i
    FgProduct qr = {(const float *)dy, lddy, (d->tokens - 1) * lddy + d->out_f, nullptr, 0, 0, (float *)dx, lddx, nullptr, d->tokens, d->in_f, d->out_f,
                    fg_plan(d->tokens, d->in_f, d->out_f, num_cus, d->out_f, 1).bm, 0, 0, d->seed, 1u, (uint32_t)d->in_f, (const float *)scale_bias,
                    nullptr, 0, nullptr};
    qr.a_es = fg_es(d->act_dtype);
    qr.out_bf16 = b16;
    qr.scale_bf16 = d->coef_dtype == RDB_BF16;
    return fg_launch<FG_KCONT, FG_NOISE_1D>(qr, num_cus, s, "f32_gemm_kernel (dx += s dy . R)");
}

// dcoef is overwritten (no zero fill needed).
// d_scale_bias: NULL, or where the gradient of the random bias's scale goes: <dy, x . R^T>.
int linear_dcoef_f32(float *dcoef, float *d_scale_bias, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus,
                     void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    rdb_linear_desc dd = *d;
    dd.coef_dtype = dd.act_dtype;   // no coefficients are read here
    if (!fg_ok(&dd) || !fg_wanted(&dd) || !fg_ws_ok(RDB_OP_LINEAR_BWD_DCOEF, &dd, num_cus, workspace, workspace_bytes)) return RDB_E_UNSUPPORTED;
    if (d->tokens * ldx >= (1ll << 29) || d->tokens * lddy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    float *z = (float *)workspace;
    if (int rc = fg_project(z, (const float *)x, ldx, &dd, num_cus, s)) return rc;
    // dC[out_f x k] = dy^T . z: both sides are read across their rows (the contraction runs over the tokens)
    const int zs = zt_plan(&dd, d->in_f, num_cus).ranges;
    float *part = reinterpret_cast<float *>(static_cast<char *>(workspace) + up256(d->tokens * d->k * 4) * (zs > 1 ? 1 + zs : 1));
    FgProduct q = {(const float *)dy, lddy, (d->tokens - 1) * lddy + d->out_f, z, d->k, d->tokens * d->k, dcoef, d->k, nullptr,
                   d->out_f, d->k, d->tokens, 128, 0, 0, d->seed};
    const FgPlan dcp = dc_plan(&dd, num_cus);
    q.a_es = fg_es(d->act_dtype);
    if (int rc = fg_launch_ranges<FG_MCONT, FG_MCONT>(q, dcp, part, up256(d->out_f * d->k * 4) / 4, num_cus, s, "f32_gemm_kernel (dC = dy^T . z)")) return rc;
    if (!d_scale_bias) return RDB_OK;
    // <dy, x . R^T>: the random-bias product once more, each block reducing its tile against dy's; then the blocks in order
    float *dots = part + (dcp.ranges > 1 ? (int64_t)dcp.ranges * (up256(d->out_f * d->k * 4) / 4) : 0);
    FgProduct qr = {(const float *)x, ldx, (d->tokens - 1) * ldx + d->in_f, nullptr, 0, 0, nullptr, 0, nullptr, d->tokens, d->out_f, d->in_f,
                    fg_plan(d->tokens, d->out_f, d->in_f, num_cus, d->in_f, 1).bm, 0, 0, d->seed, (uint32_t)d->in_f, 1u, nullptr,
                    (const float *)dy, lddy, dots};
    qr.a_es = fg_es(d->act_dtype);
    qr.out_bf16 = d->act_dtype == RDB_BF16;   // dy, the matrix the product is reduced against
    if (int rc = fg_launch<FG_KCONT, FG_NOISE_1D>(qr, num_cus, s, "f32_gemm_kernel (<dy, x . R^T>)")) return rc;
    const int nblocks = (int)(cdiv(d->tokens, qr.bm) * cdiv(d->out_f, FG_BN));
    f32_sum_scalars_kernel<<<1, 256, 0, s>>>(d_scale_bias, dots, nblocks);
    return check_launch("f32_sum_scalars_kernel");
}

// ----------------------------------------------------------------------------------------------- dW = dy^T . x on its own
// For the vector-coef coefficient gradient: every element of dW meets k hashed values, so that gradient is bound by the hash
// whatever is fused into it, and a kernel that forms dW tile by tile per block of tokens repeats the k hashes per element for
// every block.  With room for dW (fp32, [out_f x in_f]) in the caller's workspace it is formed once, by this product, and
// contracted once by the kernels of rdb_materialize_bwd.  Scratch behind dW: one more [out_f x in_f] matrix per token range.
static FgPlan dw_plan(const rdb_linear_desc *d, int num_cus) { return fg_plan(d->out_f, d->in_f, d->tokens, num_cus, 256, 64); }
int64_t linear_dw_f32_workspace(const rdb_linear_desc *d, int num_cus)
{
    if (d->out_f * d->in_f >= (1ll << 29) || d->tokens <= 0) return 0;
    const int r = dw_plan(d, num_cus).ranges;
    return up256(d->out_f * d->in_f * 4) * (1 + (r > 1 ? r : 0));
}
int linear_dw_f32(float *dW, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    if (d->tokens * lddy >= (1ll << 29) || d->tokens * ldx >= (1ll << 29) || d->out_f * d->in_f >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    FgProduct q = {(const float *)dy, lddy, (d->tokens - 1) * lddy + d->out_f, (const float *)x, ldx, (d->tokens - 1) * ldx + d->in_f, dW, d->in_f, nullptr,
                   d->out_f, d->in_f, d->tokens, 128, 0, 0, d->seed};
    q.a_es = q.b_es = fg_es(d->act_dtype);
    const int64_t stride = up256(d->out_f * d->in_f * 4) / 4;
    return fg_launch_ranges<FG_MCONT, FG_MCONT>(q, dw_plan(d, num_cus), dW + stride, stride, num_cus, s, "f32_gemm_kernel (dW = dy^T . x)");
}

// ----------------------------------------------------------------------------------------------- projected form in fp32
// What a training step keeps from the forward to the backward pass (all that the latter needs of x): z = x . N^T in fp32, [tokens x k] row-major,
// behind a 256-byte header (the same role as the bf16 state of rdb_direct.hpp; no fragment orders, no transposed copies: these
// kernels stage both operands through LDS).  fp32 activations and coefficients, one launch's worth of tokens.
static bool fg_state_ok(const rdb_linear_desc *d)
{
    return d->act_dtype == RDB_F32 && d->coef_dtype == RDB_F32 && fg_ok(d) && d->tokens * std::max(d->in_f, d->out_f) < (1ll << 28);
}
int64_t linear_f32_state_bytes(const rdb_linear_desc *d) { return fg_state_ok(d) ? 256 + up256(d->tokens * d->k * 4) : 0; }
static float *fg_state_z(const void *state) { return reinterpret_cast<float *>(static_cast<char *>(const_cast<void *>(state)) + 256); }

// workspace of the backward pass from the state: t = dy . C with the partial matrices of its ranges, then the partial matrices
// of dC = dy^T . z
int64_t linear_f32_bwd_projected_workspace(const rdb_linear_desc *d, int num_cus)
{
    if (!fg_state_ok(d)) return 0;
    const int r = dc_plan(d, num_cus).ranges;
    return linear_f32_workspace(RDB_OP_LINEAR_BWD_DX, d, num_cus) + (r > 1 ? (int64_t)r * up256(d->out_f * d->k * 4) : 0);
}

static int fg_fwd_from_z(void *y, int64_t ldy, const float *z, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus, hipStream_t s)
{
    FgProduct q = {z, d->k, d->tokens * d->k, (const float *)coef, d->k, d->out_f * d->k, (float *)y, ldy, (const float *)bias,
                   d->tokens, d->out_f, d->k, fg_plan(d->tokens, d->out_f, d->k, num_cus, d->k, 1).bm, 0, 0, d->seed};
    return fg_launch<FG_KCONT, FG_KCONT>(q, num_cus, s, "f32_gemm_kernel (y = z . C^T)");
}

// state <- z.  The partial matrices of the projection's contraction ranges need scratch that this call is not given: with y
// they lie in y's memory, which is written last (only when y is contiguous, and as many ranges as fit there); without y the
// contraction runs in one range.
int linear_project_f32(void *state, void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *bias, const rdb_linear_desc *d,
                       int num_cus, hipStream_t s)
{
    if (!fg_state_ok(d) || !fg_aligned16(state) || d->tokens * ldx >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    if (y && (d->tokens * ldy >= (1ll << 29))) return RDB_E_UNSUPPORTED;
    float *z = fg_state_z(state);
    float *part = nullptr;
    int max_ranges = 1;
    if (y && ldy == d->out_f && fg_aligned16(y)) {
        part = (float *)y;
        max_ranges = (int)((d->tokens * d->out_f * 4) / up256(d->tokens * d->k * 4));
    }
    if (int rc = fg_project(z, (const float *)x, ldx, d, num_cus, s, part ? part : z, max_ranges)) return rc;
    if (!y) return RDB_OK;
    return fg_fwd_from_z(y, ldy, z, coef, bias, d, num_cus, s);
}

int linear_fwd_projected_f32(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                             hipStream_t s)
{
    if (!fg_state_ok(d) || d->tokens * ldy >= (1ll << 29)) return RDB_E_UNSUPPORTED;
    return fg_fwd_from_z(y, ldy, fg_state_z(state), coef, bias, d, num_cus, s);
}

// dx (NULL: not wanted) and dcoef from dy, the state and C.
int linear_bwd_projected_f32(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *state, const void *coef,
                             const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s)
{
    if (!fg_state_ok(d) || !workspace || !fg_aligned16(workspace) || workspace_bytes < linear_f32_bwd_projected_workspace(d, num_cus))
        return RDB_E_UNSUPPORTED;
    if (d->tokens * lddy >= (1ll << 29) || (dx && d->tokens * lddx >= (1ll << 29))) return RDB_E_UNSUPPORTED;
    if (dx) {
        if (int rc = linear_dx_f32(dx, lddx, dy, lddy, coef, nullptr, d, num_cus, workspace, workspace_bytes, s)) return rc;
    }
    float *part = reinterpret_cast<float *>(static_cast<char *>(workspace) + linear_f32_workspace(RDB_OP_LINEAR_BWD_DX, d, num_cus));
    FgProduct q = {(const float *)dy, lddy, (d->tokens - 1) * lddy + d->out_f, fg_state_z(state), d->k, d->tokens * d->k, dcoef, d->k, nullptr,
                   d->out_f, d->k, d->tokens, 128, 0, 0, d->seed};
    return fg_launch_ranges<FG_MCONT, FG_MCONT>(q, dc_plan(d, num_cus), part, up256(d->out_f * d->k * 4) / 4, num_cus, s,
                                                "f32_gemm_kernel (dC = dy^T . z)");
}

// ----------------------------------------------------------------------------------------------- materialise on the matrix cores
// W = C . N (+ s . R) written to memory as fp32, matrix-coef, the (coef_rows, row_len) base tensor or its transpose
// (src/rten_cpp/RandumbTensor.py:235-290), and its adjoint dcoef = dW . N^T (RandumbTensor.py:304-359): the same products as
// the factored layer's, with the other operand being C or dW.  Worth it from some tens of millions of multiply-adds on; below
// that the caller's vector-ALU kernels are as fast.
constexpr int64_t FG_MATERIALIZE_MIN_MACS = (int64_t)1 << 26, FG_COEF_GRAD_MIN_MACS = (int64_t)1 << 23;

static bool fg_mat_ok(int64_t coef_rows, int64_t k, int64_t row_len, int64_t min_macs)
{
    return coef_rows > 0 && k > 0 && row_len > 0 && coef_rows * k < (1ll << 29) && coef_rows * row_len < (1ll << 29) && row_len < (1 << 30) &&
           coef_rows * k * row_len >= min_macs;
}

int materialize_mat_f32(float *out, const void *coef, int coef_dtype, int64_t coef_rows, int64_t k, int64_t row_len, bool transposed, uint32_t seed,
                        const void *scale_bias, int num_cus, hipStream_t s)
{
    if (!fg_mat_ok(coef_rows, k, row_len, FG_MATERIALIZE_MIN_MACS)) return RDB_E_UNSUPPORTED;
    const float *C = (const float *)coef;
    if (!transposed) {
        // W[o, i] = sum_m C[o, m] noise(i, m): rows = o from C, columns = i hashed; the random bias at index o * row_len + i
        FgProduct q = {C, k, coef_rows * k, nullptr, 0, 0, out, row_len, nullptr, coef_rows, row_len, k,
                       fg_plan(coef_rows, row_len, k, num_cus, k, 1).bm, 0, 0, seed, (uint32_t)row_len, 1u, (const float *)scale_bias, nullptr, 0, nullptr};
        q.a_es = fg_es(coef_dtype);
        q.scale_bf16 = coef_dtype == RDB_BF16;
            return fg_launch<FG_KCONT, FG_NOISE_I>(q, num_cus, s, "f32_gemm_kernel (W = C . N)");
    }
    // W^T[i, o]: rows = i hashed, columns = o from C; the random bias at index o * row_len + i
    FgProduct q = {nullptr, 0, 0, C, k, coef_rows * k, out, coef_rows, nullptr, row_len, coef_rows, k,
                   fg_plan(row_len, coef_rows, k, num_cus, k, 1).bm, 0, 0, seed, 1u, (uint32_t)row_len, (const float *)scale_bias, nullptr, 0, nullptr};
    q.b_es = fg_es(coef_dtype);
    q.scale_bf16 = coef_dtype == RDB_BF16;
    return fg_launch<FG_NOISE_I, FG_KCONT>(q, num_cus, s, "f32_gemm_kernel (W^T = N^T . C^T)");
}

static FgPlan mat_bwd_plan(int64_t coef_rows, int64_t k, int64_t row_len, int num_cus) { return fg_plan(coef_rows, k, row_len, num_cus, 256, 64); }

// scratch of the adjoint: one [coef_rows x k] matrix per range of the row (none with a single range)
int64_t coef_grad_mat_f32_workspace(int64_t coef_rows, int64_t k, int64_t row_len, int num_cus)
{
    if (!fg_mat_ok(coef_rows, k, row_len, FG_COEF_GRAD_MIN_MACS)) return 0;
    const int r = mat_bwd_plan(coef_rows, k, row_len, num_cus).ranges;
    return r > 1 ? (int64_t)r * up256(coef_rows * k * 4) : 0;
}

// dcoef[o, m] = sum_i dW[o, i] noise(i, m); dcoef is overwritten
int coef_grad_mat_f32(float *dcoef, const void *dW, int dw_dtype, int64_t coef_rows, int64_t k, int64_t row_len, uint32_t seed, void *workspace,
                      int64_t workspace_bytes, int num_cus, hipStream_t s)
{
    if (!fg_mat_ok(coef_rows, k, row_len, FG_COEF_GRAD_MIN_MACS)) return RDB_E_UNSUPPORTED;
    const int64_t need = coef_grad_mat_f32_workspace(coef_rows, k, row_len, num_cus);
    if (need > 0 && (!workspace || !fg_aligned16(workspace) || workspace_bytes < need)) return RDB_E_UNSUPPORTED;
    FgProduct q = {(const float *)dW, row_len, coef_rows * row_len, nullptr, 0, 0, dcoef, k, nullptr, coef_rows, k, row_len, 128, 0, 0, seed};
    q.a_es = fg_es(dw_dtype);
    return fg_launch_ranges<FG_KCONT, FG_NOISE_M>(q, mat_bwd_plan(coef_rows, k, row_len, num_cus), (float *)workspace, up256(coef_rows * k * 4) / 4, num_cus,
                                                  s, "f32_gemm_kernel (dcoef = dW . N^T)");
}

}  // namespace rdb
