// Fused linear layer on a pseudorandom weight, general-shape kernels ("tile" algorithm).
//
//   forward : y  = x  . W^T        W (out_f x in_f) is regenerated block by block in LDS
//   bwd dx  : dx = dy . W
//   bwd dC  : dW = dy^T . x  is produced block by block in registers and contracted at once with the
//             regenerated noise, dcoef += dW . Noise^T; neither W nor dW is ever written to memory.
//
// Each 256-thread block owns a 128 x 128 output block (4 waves, 64 x 64 each, 32x32 MFMA blocks) and walks the
// contraction in steps of 32.  Reference behaviour replaced: materialize() + dense product per aten.mm
// (src/rten_cpp/RandumbTensor.py:942-952, 771-791), autograd's MmBackward on the dense weight, and
// RandumbTensorConstructor.backward -> materialize_bwd / scale_bias_bwd (RandumbTensor.py:979-990).
#include <algorithm>

#include "rdb_direct.hpp"
#include "rdb_tile.hpp"

namespace rdb {

constexpr int BM = 128, BN = 128, BK = 32;

struct LinParams {
    WeightSpec w;
    const void *a;  // fwd: x, dx: dy, dcoef: dy
    const void *b;  // dcoef: x
    void *out;      // fwd: y, dx: dx
    const void *bias;
    float *dcoef;
    float *dsb;
    int64_t lda, ldb, ldo;
    int64_t tokens;
    int vec_a, vec_b;  // 16-byte vector loads allowed
};

template <typename T>
__device__ __forceinline__ void mma_step(f32x16 (&acc)[2][2], const T *As, const T *Bs, int ld, int wm, int wn, int r, int g)
{
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
        typename MMA<T>::Frag fa[2], fb[2];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) fa[mi] = MMA<T>::load(As + (wm * 64 + mi * 32 + r) * ld + ks * 16 + g * 8);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) fb[ni] = MMA<T>::load(Bs + (wn * 64 + ni * 32 + r) * ld + ks * 16 + g * 8);
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) MMA<T>::mma(acc[mi][ni], fa[mi], fb[ni]);
    }
}

// out[(m0+m)*ldo + n0+n] = acc (+ bias[n]) for the block's valid part.
template <typename T>
__device__ __forceinline__ void store_block(const f32x16 (&acc)[2][2], T *out, int64_t ldo, int64_t m0, int64_t M, int64_t n0,
                                            int64_t N, const T *bias, int wm, int wn, int r, int g)
{
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
        const int64_t n = n0 + wn * 64 + ni * 32 + r;
        if (n >= N) continue;
        const float bv = bias ? to_f32<T>(bias[n]) : 0.0f;
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int64_t m = m0 + wm * 64 + mi * 32 + 8 * (j / 4) + 4 * g + (j % 4);
                if (m < M) out[m * ldo + n] = from_f32<T>(acc[mi][ni][j] + bv);
            }
    }
}

// ----------------------------------------------------------------------------------------------- forward
// y[t, o] = sum_i x[t, i] * W[o, i].  M = tokens, N = out_f, contraction over in_f.
template <typename T, bool MATRIX>
__global__ __launch_bounds__(TILE_THREADS) void linear_fwd_kernel(LinParams p)
{
    constexpr int LD = BK + MMA<T>::PAD;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);
    T *Bs = As + BM * LD;
    T *scratch = Bs + BN * LD;
    const int t = threadIdx.x, wave = t / 64, lane = t % 64, r = lane % 32, g = lane / 32, wm = wave / 2, wn = wave % 2;
    const int64_t n0 = (int64_t)blockIdx.x * BN, m0 = (int64_t)blockIdx.y * BM;
    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = zero16();
    for (int64_t k0 = 0; k0 < p.w.in_f; k0 += BK) {
        load_tile_rowmajor<T, BM, BK>(As, LD, (const T *)p.a, p.lda, m0, p.tokens, k0, p.w.in_f, p.vec_a);
        gen_w_tile<T, BN, BK, true, MATRIX>(Bs, LD, scratch, p.w, n0, k0);  // Bs[o][i]
        __syncthreads();
        mma_step<T>(acc, As, Bs, LD, wm, wn, r, g);
        __syncthreads();
    }
    store_block<T>(acc, (T *)p.out, p.ldo, m0, p.tokens, n0, p.w.out_f, (const T *)p.bias, wm, wn, r, g);
}

// ----------------------------------------------------------------------------------------------- backward dx
// dx[t, i] = sum_o dy[t, o] * W[o, i].  M = tokens, N = in_f, contraction over out_f.
template <typename T, bool MATRIX>
__global__ __launch_bounds__(TILE_THREADS) void linear_dx_kernel(LinParams p)
{
    constexpr int LD = BK + MMA<T>::PAD;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);
    T *Bs = As + BM * LD;
    T *scratch = Bs + BN * LD;
    const int t = threadIdx.x, wave = t / 64, lane = t % 64, r = lane % 32, g = lane / 32, wm = wave / 2, wn = wave % 2;
    const int64_t n0 = (int64_t)blockIdx.x * BN, m0 = (int64_t)blockIdx.y * BM;
    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = zero16();
    for (int64_t k0 = 0; k0 < p.w.out_f; k0 += BK) {
        load_tile_rowmajor<T, BM, BK>(As, LD, (const T *)p.a, p.lda, m0, p.tokens, k0, p.w.out_f, p.vec_a);
        gen_w_tile<T, BK, BN, false, MATRIX>(Bs, LD, scratch, p.w, k0, n0);  // Bs[i][o]
        __syncthreads();
        mma_step<T>(acc, As, Bs, LD, wm, wn, r, g);
        __syncthreads();
    }
    store_block<T>(acc, (T *)p.out, p.ldo, m0, p.tokens, n0, p.w.in_f, (const T *)nullptr, wm, wn, r, g);
}

// ----------------------------------------------------------------------------------------------- backward dcoef
// dW[o, i] = sum_t dy[t, o] * x[t, i] for the block (M = out_f, N = in_f, contraction over tokens), then
//   matrix-coef: dC[o, m]  += sum_i dW[o, i] * noise(i, m)           (matrix cores, m in chunks of 32)
//   vector-coef: dcoef[m]  += sum_{o,i} dW[o, i] * noise(o*sO + i*sI, m)   (vector ALU)
//   d_scale_bias           += sum_{o,i} dW[o, i] * noise(o*sO + i*sI)
// dW is rounded to T once before the contraction (a bf16 dense product would have stored it as bf16).
template <typename T, bool MATRIX>
__global__ __launch_bounds__(TILE_THREADS) void linear_dcoef_kernel(LinParams p)
{
    constexpr int LD = BK + MMA<T>::PAD;
    constexpr int LDW = BN + MMA<T>::PAD;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);
    T *Bs = As + BM * LD;
    const int t = threadIdx.x, wave = t / 64, lane = t % 64, r = lane % 32, g = lane / 32, wm = wave / 2, wn = wave % 2;
    const int64_t n0 = (int64_t)blockIdx.x * BN, m0 = (int64_t)blockIdx.y * BM;  // n0: first i, m0: first o
    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = zero16();
    for (int64_t k0 = 0; k0 < p.tokens; k0 += BK) {
        load_tile_transposed<T, BM, BK>(As, LD, (const T *)p.a, p.lda, m0, p.w.out_f, k0, p.tokens, p.vec_a);  // As[o][t]
        load_tile_transposed<T, BN, BK>(Bs, LD, (const T *)p.b, p.ldb, n0, p.w.in_f, k0, p.tokens, p.vec_b);   // Bs[i][t]
        __syncthreads();
        mma_step<T>(acc, As, Bs, LD, wm, wn, r, g);
        __syncthreads();
    }
    // stage dW as Ws[o][i] (i contiguous); entries outside the matrix are exact zeros (zero-filled operands)
    T *Ws = reinterpret_cast<T *>(smem_raw);  // [BM][LDW], reuses the operand tiles
    T *Ns = Ws + BM * LDW;                    // [32][LDW]  Ns[m][i]
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int o = wm * 64 + mi * 32 + 8 * (j / 4) + 4 * g + (j % 4), i = wn * 64 + ni * 32 + r;
                Ws[o * LDW + i] = from_f32<T>(acc[mi][ni][j]);
            }
    __syncthreads();
    const WeightSpec &w = p.w;
    if constexpr (MATRIX) {
        // E[a = m][b = o] = sum_i Ns[m][i] * Ws[o][i]; wave `wave` owns o-block `wave` (32 rows of the tile)
        for (int64_t mc = 0; mc < w.k; mc += 32) {
            for (int e = t; e < 32 * BN; e += TILE_THREADS) {
                const int mm = e / BN, ii = e % BN;
                Ns[mm * LDW + ii] = from_f32<T>(noise2d((uint32_t)(n0 + ii), (uint32_t)(mc + mm), w.seed));
            }
            __syncthreads();
            f32x16 e16 = zero16();
#pragma unroll
            for (int ks = 0; ks < BN / 16; ++ks) {
                typename MMA<T>::Frag fa = MMA<T>::load(Ns + r * LDW + ks * 16 + g * 8);
                typename MMA<T>::Frag fb = MMA<T>::load(Ws + (wave * 32 + r) * LDW + ks * 16 + g * 8);
                MMA<T>::mma(e16, fa, fb);
            }
            const int64_t o = m0 + wave * 32 + r;
            if (o < w.out_f) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int64_t m = mc + 8 * (j / 4) + 4 * g + (j % 4);
                    if (m < w.k) unsafeAtomicAdd(p.dcoef + o * w.k + m, e16[j]);
                }
            }
            __syncthreads();
        }
    } else {
        // thread (ml = t % 32, grp = t / 32): coefficient mc + ml, elements grp, grp + 8, ... of the block
        float *red = reinterpret_cast<float *>(Ns);  // [8][32]
        const int ml = t % 32, grp = t / 32;
        for (int64_t mc = 0; mc < w.k; mc += 32) {
            const uint32_t mterm = (uint32_t)(mc + ml) * SQ5_N1 + w.seed;
            float s = 0.0f;
            for (int e = grp; e < BM * BN; e += 8) {
                const int oo = e / BN, ii = e % BN;
                const uint32_t a = (uint32_t)((m0 + oo) * w.sO + (n0 + ii) * w.sI);
                s = fmaf(sq5_unit(sq5_tail(a * PN1 + mterm)), to_f32<T>(Ws[oo * LDW + ii]), s);
            }
            __syncthreads();
            red[grp * 32 + ml] = s;
            __syncthreads();
            if (grp == 0 && mc + ml < w.k) {
                float tot = red[ml];
#pragma unroll
                for (int j = 1; j < 8; ++j) tot += red[j * 32 + ml];
                unsafeAtomicAdd(p.dcoef + mc + ml, tot);
            }
        }
    }
    if (p.dsb) {
        float s = 0.0f;
        for (int e = t; e < BM * BN; e += TILE_THREADS) {
            const int oo = e / BN, ii = e % BN;
            s = fmaf(to_f32<T>(Ws[oo * LDW + ii]), noise1d((uint32_t)((m0 + oo) * w.sO + (n0 + ii) * w.sI), w.seed), s);
        }
        __syncthreads();
        float *red = reinterpret_cast<float *>(Ns);
        red[t] = s;
        __syncthreads();
        for (int st = TILE_THREADS / 2; st > 0; st >>= 1) {
            if (t < st) red[t] += red[t + st];
            __syncthreads();
        }
        if (t == 0) unsafeAtomicAdd(p.dsb, red[0]);
    }
}

// Clears n floats.  A fill kernel rather than hipMemsetAsync so that callers can capture the launch in a HIP graph.
// 16-byte stores over the aligned middle, scalar stores on the ragged ends.
__global__ __launch_bounds__(256) void fill_zero_kernel(float *p, int64_t n)
{
    const int64_t head = ((16 - ((uintptr_t)p & 15)) & 15) / 4 < n ? ((16 - ((uintptr_t)p & 15)) & 15) / 4 : n;
    const int64_t nvec = (n - head) / 4, tail = head + nvec * 4;
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x, nthr = (int64_t)gridDim.x * 256;
    f32x4 *v = reinterpret_cast<f32x4 *>(p + head);
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t e = tid; e < nvec; e += nthr) v[e] = zero;
    if (tid < head) p[tid] = 0.0f;
    if (tid < n - tail) p[tail + tid] = 0.0f;
}
static int fill_zero(float *p, int64_t n, hipStream_t s)
{
    const int64_t blocks = cdiv(cdiv(n, 4) + 8, 256);
    fill_zero_kernel<<<(unsigned)(blocks < 2048 ? blocks : 2048), 256, 0, s>>>(p, n);
    return check_launch("fill_zero_kernel");
}

// ----------------------------------------------------------------------------------------------- host side
template <typename T> static size_t smem_fwd() { return sizeof(T) * ((BM + BN) * (BK + MMA<T>::PAD) + gen_scratch_elems<T, BN, BK>()); }
template <typename T> static size_t smem_dcoef()
{
    const size_t a = sizeof(T) * (BM + BN) * (BK + MMA<T>::PAD);
    const size_t b = sizeof(T) * (BM + 32) * (BN + MMA<T>::PAD);
    return a > b ? a : b;
}

static int check_desc(const char *who, const rdb_linear_desc *d)
{
    if (!d) return set_error(RDB_E_NULL, "%s: desc is NULL", who);
    if (d->tokens < 0 || d->in_f < 0 || d->out_f < 0 || d->k < 0)
        return set_error(RDB_E_SHAPE, "%s: negative size tokens=%lld in=%lld out=%lld k=%lld", who, (long long)d->tokens,
                         (long long)d->in_f, (long long)d->out_f, (long long)d->k);
    if (d->act_dtype != RDB_F32 && d->act_dtype != RDB_BF16) return set_error(RDB_E_DTYPE, "%s: unknown act dtype %d", who, d->act_dtype);
    if (d->coef_dtype != RDB_F32 && d->coef_dtype != RDB_BF16) return set_error(RDB_E_DTYPE, "%s: unknown coef dtype %d", who, d->coef_dtype);
    if (d->coef_rows != 0 && d->coef_rows != d->out_f)
        return set_error(RDB_E_SHAPE, "%s: coef_rows must be 0 or out_f (%lld), got %lld", who, (long long)d->out_f, (long long)d->coef_rows);
    if (d->coef_rows != 0 && (d->sO != d->in_f || d->sI != 1))
        return set_error(RDB_E_SHAPE, "%s: matrix-coef needs strides (in_f, 1), got (%lld, %lld)", who, (long long)d->sO, (long long)d->sI);
    if (d->sO < 0 || d->sI < 0) return set_error(RDB_E_SHAPE, "%s: negative weight stride", who);
    if (d->algo != RDB_ALGO_AUTO && d->algo != RDB_ALGO_TILE && d->algo != RDB_ALGO_STRIP && d->algo != RDB_ALGO_FACTORED)
        return set_error(RDB_E_UNSUPPORTED, "%s: unknown algo %d", who, d->algo);
    if (d->tokens > (1ll << 31) * BM || d->in_f > (1ll << 31) || d->out_f > (1ll << 31))
        return set_error(RDB_E_SHAPE, "%s: dimension too large", who);
    return RDB_OK;
}

// rdb_strip.hip
int linear_fwd_strip(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                     const rdb_linear_desc *d, int num_cus, hipStream_t s);

// rdb_factored.hip
int64_t linear_projection_bytes(const rdb_linear_desc *d);
int linear_project(void *state, const void *x, int64_t ldx, const void *coef, const rdb_linear_desc *d, hipStream_t s);
int linear_project_fwd(void *y, int64_t ldy, void *state, const void *x, int64_t ldx, const void *coef, bool with_ct, const void *bias,
                       const rdb_linear_desc *d, int num_cus, hipStream_t s);
int linear_fwd_projected(void *y, int64_t ldy, const void *z, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                         hipStream_t s);
int linear_dcoef_projected(float *dcoef, const void *dy, int64_t lddy, const void *z, const rdb_linear_desc *d, int num_cus, hipStream_t s);
int linear_fwd_factored(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                        const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dcoef_factored(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus,
                          void *workspace, int64_t workspace_bytes, hipStream_t s);

// rdb_dxstrip.hip
int linear_dx_nstrip(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                     hipStream_t s);

// rdb_smallk.hip
int64_t linear_smallk_workspace(const rdb_linear_desc *d);
int linear_fwd_smallk(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                      const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dx_smallk(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                     void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dcoef_smallk(float *dcoef, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, void *workspace,
                        int64_t workspace_bytes, hipStream_t s);

// rdb_error.hip
int num_compute_units();   // of the current device (256 when there is none)

// rdb_f32.hip
int64_t linear_f32_workspace(int op, const rdb_linear_desc *d, int num_cus);
int linear_fwd_f32(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                   const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dx_f32(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                  int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);
int64_t linear_f32_state_bytes(const rdb_linear_desc *d);
int64_t linear_f32_bwd_projected_workspace(const rdb_linear_desc *d, int num_cus);
int64_t linear_dw_f32_workspace(const rdb_linear_desc *d, int num_cus);
int linear_dw_f32(float *dW, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus, hipStream_t s);
int linear_project_f32(void *state, void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *bias, const rdb_linear_desc *d,
                       int num_cus, hipStream_t s);
int linear_fwd_projected_f32(void *y, int64_t ldy, const void *state, const void *coef, const void *bias, const rdb_linear_desc *d, int num_cus,
                             hipStream_t s);
int linear_bwd_projected_f32(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *state, const void *coef,
                             const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dcoef_f32(float *dcoef, float *d_scale_bias, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d, int num_cus,
                     void *workspace, int64_t workspace_bytes, hipStream_t s);
// rdb_dx.hip
int linear_bwd_projected(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *z, const void *coef,
                         const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, bool accumulate, bool dc_bf16,
                         hipStream_t s);
int64_t linear_dx_factored_workspace(const rdb_linear_desc *d);
int64_t linear_bwd_projected_workspace(const rdb_linear_desc *d, int num_cus, bool force_partial);
int linear_dx_factored(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias,
                       const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);

// rdb_big.hip
void set_big_tiles_mode(int mode);
int big_tiles_mode();
bool big_bwd_applies(const rdb_linear_desc *d, int num_cus);
int linear_bwd_big(void *t, float *dc, const void *dy, int64_t lddy, const void *state, const void *coef, const rdb_linear_desc *d, int num_cus,
                   bool want_t, bool want_dc, hipStream_t s);

// rdb_rbias.hip
int linear_dx_rbias_add(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *scale_bias, const rdb_linear_desc *d, hipStream_t s);
int linear_fwd_rbias_add(void *y, int64_t ldy, const void *x, int64_t ldx, const void *scale_bias, const rdb_linear_desc *d, hipStream_t s);
int64_t linear_dx_rbias_dot_floats(const rdb_linear_desc *d);
int linear_dx_rbias_add_dscale(void *dx, int64_t lddx, float *dscale, float *dot_part, const void *dy, int64_t lddy, const void *x, int64_t ldx,
                               const void *scale_bias, const rdb_linear_desc *d, hipStream_t s);

// rdb_vecsplit.hip
int64_t linear_vecsplit_workspace(int op, const rdb_linear_desc *d);
int linear_fwd_vecsplit(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias, const void *bias,
                        const rdb_linear_desc *d, int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);
int linear_dx_vecsplit(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias, const rdb_linear_desc *d,
                       int num_cus, void *workspace, int64_t workspace_bytes, hipStream_t s);

// rdb_dcoef.hip
int linear_dcoef_fast(float *dcoef, float *dsb, const void *dy, int64_t lddy, const void *x, int64_t ldx, const rdb_linear_desc *d,
                      int num_cus, hipStream_t s);

// Compute units of the current device (cached per device id).

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

static WeightSpec make_spec(const rdb_linear_desc *d, const void *coef, const void *scale_bias)
{
    WeightSpec w;
    w.coef = coef;
    w.scale_bias = scale_bias;
    w.out_f = d->out_f;
    w.in_f = d->in_f;
    w.k = d->k;
    w.sO = d->sO;
    w.sI = d->sI;
    w.seed = d->seed;
    w.coef_dtype = d->coef_dtype;
    return w;
}

template <typename K> static int launch(K kernel, dim3 grid, size_t smem, hipStream_t s, const LinParams &p, const char *name)
{
    if (smem > 48 * 1024) {
        if (int rl = reserve_lds(reinterpret_cast<const void *>(kernel), smem, name)) return rl;
    }
    kernel<<<grid, TILE_THREADS, smem, s>>>(p);
    return check_launch(name);
}

}  // namespace rdb

using namespace rdb;

static int64_t bwd_projected_workspace(const rdb_linear_desc *d, bool force_partial);

// vector-coef coefficient gradient in two passes: dW = dy^T . x into the workspace (and the partial matrices of its token
// ranges), then the contraction of rdb_materialize_bwd and, for the scale's gradient, of rdb_scale_bias_bwd, with their scratch
// behind it.  Only for a weight that is contiguous in memory (element (o, i) at o * in_f + i).
static bool vec_dcoef_two_pass_ok(const rdb_linear_desc *d)
{
    return d->coef_rows == 0 && d->sO == d->in_f && d->sI == 1 && d->k > 0 && d->tokens > 0 && d->out_f * d->in_f < (1ll << 29) &&
           (d->act_dtype == RDB_F32 || d->act_dtype == RDB_BF16);
}
static int64_t vec_dcoef_workspace(const rdb_linear_desc *d)
{
    if (!vec_dcoef_two_pass_ok(d)) return 0;
    const int64_t dw = linear_dw_f32_workspace(d, num_compute_units());
    if (dw <= 0) return 0;
    const int64_t nw = d->out_f * d->in_f;
    return dw + (rdb_materialize_bwd_workspace_bytes(0, d->k, 0, nw) + 255) / 256 * 256 + (rdb_scale_bias_bwd_workspace_bytes(nw) + 255) / 256 * 256;
}

static int64_t linear_workspace_bytes_main(int op, const rdb_linear_desc *d);

extern "C" int64_t rdb_linear_workspace_bytes(int op, const rdb_linear_desc *d)
{
    if (!d) return 0;
    int64_t need = linear_workspace_bytes_main(op, d);
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16 && d->coef_rows != 0 &&
        (op == RDB_OP_LINEAR_FWD || op == RDB_OP_LINEAR_BWD_DX || op == RDB_OP_LINEAR_BWD_DCOEF)) {
        // bf16 with a few tokens: the vector-ALU kernels of rdb_smallk.hip come first (their scratch: partial [tokens x k] matrices)
        rdb_linear_desc dd = *d;
        if (op == RDB_OP_LINEAR_BWD_DCOEF) dd.coef_dtype = RDB_BF16;
        const int64_t few = linear_smallk_workspace(&dd);
        if (few > need) need = few;
    }
    return need;
}

static int64_t linear_workspace_bytes_main(int op, const rdb_linear_desc *d)
{
    if (d->algo == RDB_ALGO_TILE || d->algo == RDB_ALGO_STRIP) return 0;
    if (d->coef_rows == 0) {   // vector-coef: the chunks' partial outputs; for the coefficient gradient dW and what its contraction needs
        if (d->algo != RDB_ALGO_AUTO) return 0;
        if (op == RDB_OP_LINEAR_BWD_DCOEF) return vec_dcoef_workspace(d);
        return linear_vecsplit_workspace(op, d);
    }
    if (d->act_dtype == RDB_F32) {  // fp32: the small-k kernels, whose scratch is one [tokens x k] fp32 matrix
        rdb_linear_desc dd = *d;
        if (op == RDB_OP_LINEAR_BWD_DCOEF) dd.coef_dtype = RDB_F32;
        if (op == RDB_OP_LINEAR_BWD_PROJECTED || op == RDB_OP_LINEAR_BWD_PROJECTED_TO) return linear_f32_bwd_projected_workspace(d, num_compute_units());
        if (op != RDB_OP_LINEAR_FWD && op != RDB_OP_LINEAR_BWD_DX && op != RDB_OP_LINEAR_BWD_DCOEF) return 0;
        // or the matrix-core kernels of rdb_f32.hip: a [tokens x k] matrix, and the coefficient gradient's token-range sums
        const int64_t a = linear_smallk_workspace(&dd), b = linear_f32_workspace(op, &dd, num_compute_units());
        return a > b ? a : b;
    }
    if (d->act_dtype == RDB_BF16 && d->coef_rows != 0 && (d->in_f % 8 || d->out_f % 8 || d->k % 8) &&
        (op == RDB_OP_LINEAR_FWD || op == RDB_OP_LINEAR_BWD_DX || op == RDB_OP_LINEAR_BWD_DCOEF)) {
        // bf16 layers the bf16 factored kernels do not take (sizes that are not multiples of 8): the fp32 matrix-core kernels
        // with bf16 matrices read value by value
        rdb_linear_desc dd = *d;
        if (op == RDB_OP_LINEAR_BWD_DCOEF) dd.coef_dtype = RDB_BF16;
        return linear_f32_workspace(op, &dd, num_compute_units());
    }
    if (op == RDB_OP_LINEAR_BWD_DX) return linear_dx_factored_workspace(d);
    if (op == RDB_OP_LINEAR_BWD_DX_DSCALE) {   // dy.C, then one float per tile of the random-bias product
        const int64_t t = linear_dx_factored_workspace(d);
        return t > 0 ? (t + 255) / 256 * 256 + linear_dx_rbias_dot_floats(d) * 4 : 0;
    }
    if (op == RDB_OP_LINEAR_RBIAS_BWD)   // one float per tile of the random-bias product (the gradient of the scale)
        return (d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16 && d->in_f % 8 == 0 && d->out_f % 8 == 0) ? linear_dx_rbias_dot_floats(d) * 4 : 0;
    if (op == RDB_OP_LINEAR_BWD_PROJECTED) return bwd_projected_workspace(d, false);
    if (op == RDB_OP_LINEAR_BWD_PROJECTED_TO) return bwd_projected_workspace(d, true);
    if (op == RDB_OP_LINEAR_FWD) return d->coef_dtype == RDB_BF16 ? linear_projection_bytes(d) : 0;
    if (op == RDB_OP_LINEAR_BWD_DCOEF) return linear_projection_bytes(d);  // reads no coefficients: their dtype does not matter
    return 0;
}

extern "C" int rdb_linear_fwd(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias,
                              const void *bias, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    int rc = check_desc("rdb_linear_fwd", d);
    if (rc) return rc;
    if (d->tokens == 0 || d->out_f == 0) return RDB_OK;
    if (!y || (!x && d->in_f > 0) || (!coef && d->k > 0)) return set_error(RDB_E_NULL, "rdb_linear_fwd: y, x or coef is NULL");
    if (ldy < d->out_f || ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_fwd: leading dimension smaller than the row");
    hipStream_t s = (hipStream_t)stream;
    if (d->algo == RDB_ALGO_AUTO && d->coef_rows == 0) {
        // vector-coef, up to a few thousand tokens, with room for the partial outputs: W tiles spread over all compute units
        rc = linear_fwd_vecsplit(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16 && d->tokens <= 96) {
        // a few tokens: the matrix-core kernels below would run a handful of blocks, each alone with a contraction over all of
        // in_f; the vector-ALU kernels spread it over the chip (16 tokens x 4096 -> 4096, k = 256: 39 us against 12)
        rc = linear_fwd_smallk(y, ldy, x, ldx, coef, scale_bias, bias, d, workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO || d->algo == RDB_ALGO_FACTORED) {
        rc = linear_fwd_factored(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        rc = linear_fwd_smallk(y, ldy, x, ldx, coef, scale_bias, bias, d, workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        if (d->act_dtype == RDB_F32) {
            rc = linear_fwd_f32(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), workspace, workspace_bytes, s);
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
        if (d->algo == RDB_ALGO_FACTORED)
            return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd: the factored algorithm needs matrix-coef, no scale_bias, a workspace of "
                                                "rdb_linear_workspace_bytes() bytes and either bf16 (activations and coef; sizes that are "
                                                "multiples of 8; aligned rows) or fp32 (sizes that are multiples of 4; aligned rows)");
    }
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16 && d->coef_rows != 0 && (d->in_f % 8 || d->out_f % 8 || d->k % 8)) {
        // bf16 sizes the bf16 factored kernels do not take (not multiples of 8): the fp32-accurate matrix-core kernels reading the
        // bf16 matrices, ahead of the kernel that forms weight strips on chip (4096 tokens x 1000 -> 1000, k = 100: 31 against 133 us)
        rc = linear_fwd_f32(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO && scale_bias && d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16) {
        // W = C.N + s.R: the low-rank share through the factored kernels where AUTO would take them without the random bias,
        // then the random-bias share (full rank: a product with R hashed as an operand) added on top.  Ahead of the kernel that
        // forms weight strips on chip at every size measured (8192 tokens x 768 -> 768, k = 256: 41 against 74 us; 768 -> 3072:
        // 118 against 121; 2048 tokens x 768 -> 3072: 43 against 74).
        rdb_linear_desc df = *d;
        rc = linear_fwd_factored(y, ldy, x, ldx, coef, nullptr, bias, &df, num_compute_units(), workspace, workspace_bytes, s);
        if (rc == RDB_OK) {
            rc = linear_fwd_rbias_add(y, ldy, x, ldx, scale_bias, d, s);
            if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd: internal: the random-bias share refused a request the factored share took");
        }
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo != RDB_ALGO_TILE) {
        rc = linear_fwd_strip(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        if (d->algo == RDB_ALGO_STRIP)
            return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd: the strip algorithm needs matrix-coef, bf16 activations, in_f %% 8 == 0, "
                                                "16-byte aligned x rows and a weight strip that fits LDS");
    }
    if (d->algo == RDB_ALGO_AUTO && scale_bias && d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16) {
        // the same two shares where the rule above did not take the factored form (k so long that it is not the cheaper one in
        // flops) and no weight strip fits on chip: still far ahead of the general kernel below
        rdb_linear_desc df = *d;
        df.algo = RDB_ALGO_FACTORED;
        rc = linear_fwd_factored(y, ldy, x, ldx, coef, nullptr, bias, &df, num_compute_units(), workspace, workspace_bytes, s);
        if (rc == RDB_OK) {
            rc = linear_fwd_rbias_add(y, ldy, x, ldx, scale_bias, d, s);
            if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd: internal: the random-bias share refused a request the factored share took");
        }
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16) {
        // bf16 requests that kept every kernel above away (rows that are not 16-byte aligned, ...): the same kernels, reading bf16
        // value by value
        rc = linear_fwd_f32(y, ldy, x, ldx, coef, scale_bias, bias, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    const int es = d->act_dtype == RDB_BF16 ? 2 : 4;
    LinParams p = {};
    p.w = make_spec(d, coef, scale_bias);
    p.a = x;
    p.lda = ldx;
    p.out = y;
    p.ldo = ldy;
    p.bias = bias;
    p.tokens = d->tokens;
    p.vec_a = aligned16(x) && (ldx * es) % 16 == 0;
    dim3 grid((unsigned)cdiv(d->out_f, BN), (unsigned)cdiv(d->tokens, BM));
    const bool mat = d->coef_rows != 0;
    if (d->act_dtype == RDB_BF16)
        return mat ? launch(linear_fwd_kernel<bf16_t, true>, grid, smem_fwd<bf16_t>(), s, p, "linear_fwd_kernel<bf16,matrix>")
                   : launch(linear_fwd_kernel<bf16_t, false>, grid, smem_fwd<bf16_t>(), s, p, "linear_fwd_kernel<bf16,vector>");
    return mat ? launch(linear_fwd_kernel<float, true>, grid, smem_fwd<float>(), s, p, "linear_fwd_kernel<f32,matrix>")
               : launch(linear_fwd_kernel<float, false>, grid, smem_fwd<float>(), s, p, "linear_fwd_kernel<f32,vector>");
}

extern "C" int rdb_linear_bwd_dx(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef, const void *scale_bias,
                                 const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    int rc = check_desc("rdb_linear_bwd_dx", d);
    if (rc) return rc;
    if (d->tokens == 0 || d->in_f == 0) return RDB_OK;
    if (!dx || (!dy && d->out_f > 0) || (!coef && d->k > 0)) return set_error(RDB_E_NULL, "rdb_linear_bwd_dx: dx, dy or coef is NULL");
    if (lddx < d->in_f || lddy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_bwd_dx: leading dimension smaller than the row");
    if (d->algo == RDB_ALGO_AUTO && d->coef_rows == 0) {
        rc = linear_dx_vecsplit(dx, lddx, dy, lddy, coef, scale_bias, d, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16 && d->tokens <= 96) {   // a few tokens: as in rdb_linear_fwd
        rc = linear_dx_smallk(dx, lddx, dy, lddy, coef, scale_bias, d, workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO || d->algo == RDB_ALGO_FACTORED) {
        if (scale_bias && d->act_dtype == RDB_BF16 && d->coef_dtype == RDB_BF16 && d->tokens * lddx < (1ll << 29)) {
            // W = C.N + s.R: the low-rank share through the factored kernels, then the random-bias share added on top
            rdb_linear_desc df = *d;
            df.algo = RDB_ALGO_FACTORED;   // also where it is more flops than a product on a stored W: the alternative is the general kernel
            rc = linear_dx_factored(dx, lddx, dy, lddy, coef, nullptr, &df, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
            if (rc == RDB_OK) {
                rc = linear_dx_rbias_add(dx, lddx, dy, lddy, scale_bias, d, (hipStream_t)stream);
                if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dx: internal: the random-bias share refused a request the factored share took");
            }
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
        rc = linear_dx_factored(dx, lddx, dy, lddy, coef, scale_bias, d, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        rc = linear_dx_smallk(dx, lddx, dy, lddy, coef, scale_bias, d, workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        if (d->act_dtype == RDB_F32) {
            rc = linear_dx_f32(dx, lddx, dy, lddy, coef, scale_bias, d, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
        if (d->algo == RDB_ALGO_FACTORED)
            return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dx: the factored algorithm needs matrix-coef, a workspace of "
                                                "rdb_linear_workspace_bytes() bytes and either bf16 (activations and coef; sizes that are "
                                                "multiples of 8; aligned rows) or fp32 (sizes that are multiples of 4; aligned rows)");
    }
    if (d->algo != RDB_ALGO_TILE) {  // forms W chunks on chip, with the block's noise columns hashed once
        rc = linear_dx_nstrip(dx, lddx, dy, lddy, coef, scale_bias, d, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        if (d->algo == RDB_ALGO_STRIP)
            return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dx: the strip algorithm needs matrix-coef in bf16 with k <= 256, bf16 "
                                                "activations, no scale_bias, sizes that are multiples of 8 and aligned rows");
    }
    if (d->algo == RDB_ALGO_AUTO) {
        // Nothing above took it (k > 256, say, where no kernel re-forms W for the input gradient on the matrix cores): the
        // factored form's two products are still far ahead of the general kernel below, also where they are more flops than
        // one product on a stored W would be (2048 tokens, 1024 -> 1024, k = 512, bf16: 1.06 ms for the general kernel).
        rdb_linear_desc df = *d;
        df.algo = RDB_ALGO_FACTORED;
        rc = linear_dx_factored(dx, lddx, dy, lddy, coef, scale_bias, &df, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != RDB_E_UNSUPPORTED) return rc;
        if (d->act_dtype == RDB_BF16) {   // sizes that are not multiples of 8: the fp32 matrix cores, reading bf16 value by value
            rc = linear_dx_f32(dx, lddx, dy, lddy, coef, scale_bias, d, num_compute_units(), workspace, workspace_bytes, (hipStream_t)stream);
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
    }
    const int es = d->act_dtype == RDB_BF16 ? 2 : 4;
    LinParams p = {};
    p.w = make_spec(d, coef, scale_bias);
    p.a = dy;
    p.lda = lddy;
    p.out = dx;
    p.ldo = lddx;
    p.tokens = d->tokens;
    p.vec_a = aligned16(dy) && (lddy * es) % 16 == 0;
    dim3 grid((unsigned)cdiv(d->in_f, BN), (unsigned)cdiv(d->tokens, BM));
    hipStream_t s = (hipStream_t)stream;
    const bool mat = d->coef_rows != 0;
    if (d->act_dtype == RDB_BF16)
        return mat ? launch(linear_dx_kernel<bf16_t, true>, grid, smem_fwd<bf16_t>(), s, p, "linear_dx_kernel<bf16,matrix>")
                   : launch(linear_dx_kernel<bf16_t, false>, grid, smem_fwd<bf16_t>(), s, p, "linear_dx_kernel<bf16,vector>");
    return mat ? launch(linear_dx_kernel<float, true>, grid, smem_fwd<float>(), s, p, "linear_dx_kernel<f32,matrix>")
               : launch(linear_dx_kernel<float, false>, grid, smem_fwd<float>(), s, p, "linear_dx_kernel<f32,vector>");
}

extern "C" int rdb_linear_bwd_dx_dscale(void *dx, int64_t lddx, float *d_scale_bias, const void *dy, int64_t lddy, const void *x, int64_t ldx,
                                        const void *coef, const void *scale_bias, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes,
                                        void *stream)
{
    int rc = check_desc("rdb_linear_bwd_dx_dscale", d);
    if (rc) return rc;
    if (!dx || !d_scale_bias || !dy || !x || !coef || !scale_bias)
        return set_error(RDB_E_NULL, "rdb_linear_bwd_dx_dscale: dx, d_scale_bias, dy, x, coef or scale_bias is NULL");
    if (lddx < d->in_f || lddy < d->out_f || ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_bwd_dx_dscale: leading dimension smaller than the row");
    const int64_t need = rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX_DSCALE, d), t_bytes = (linear_dx_factored_workspace(d) + 255) / 256 * 256;
    const char *why = "rdb_linear_bwd_dx_dscale: needs matrix-coef, bf16 activations and coefficients, sizes that are multiples of 8, 16-byte "
                      "aligned rows and a workspace of rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX_DSCALE) bytes";
    if (d->act_dtype != RDB_BF16 || d->coef_dtype != RDB_BF16 || d->coef_rows == 0 || need <= 0 || !workspace || workspace_bytes < need ||
        d->tokens * lddx >= (1ll << 29))
        return set_error(RDB_E_UNSUPPORTED, "%s", why);
    rdb_linear_desc df = *d;
    df.algo = RDB_ALGO_FACTORED;   // the low-rank share through the factored kernels whatever the flop counts say
    hipStream_t s = (hipStream_t)stream;
    rc = linear_dx_factored(dx, lddx, dy, lddy, coef, nullptr, &df, num_compute_units(), workspace, workspace_bytes, s);
    if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "%s", why);
    if (rc) return rc;
    float *dots = reinterpret_cast<float *>(static_cast<char *>(workspace) + t_bytes);
    rc = linear_dx_rbias_add_dscale(dx, lddx, d_scale_bias, dots, dy, lddy, x, ldx, scale_bias, d, s);
    if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "%s", why);
    return rc;
}

// The random-bias share on its own, on top of a result that holds the low-rank share already.
static int rbias_request_ok(const char *who, const rdb_linear_desc *d)
{
    if (d->act_dtype != RDB_BF16 || d->coef_dtype != RDB_BF16 || d->coef_rows == 0 || d->in_f % 8 || d->out_f % 8)
        return set_error(RDB_E_UNSUPPORTED, "%s: needs matrix-coef, bf16 activations and coefficients, and sizes that are multiples of 8", who);
    return RDB_OK;
}

extern "C" int rdb_linear_rbias_fwd(void *y, int64_t ldy, const void *x, int64_t ldx, const void *scale_bias, const rdb_linear_desc *d, void *stream)
{
    int rc = check_desc("rdb_linear_rbias_fwd", d);
    if (rc) return rc;
    if (!y || !x || !scale_bias) return set_error(RDB_E_NULL, "rdb_linear_rbias_fwd: y, x or scale_bias is NULL");
    if (ldy < d->out_f || ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_rbias_fwd: leading dimension smaller than the row");
    if ((rc = rbias_request_ok("rdb_linear_rbias_fwd", d))) return rc;
    rc = linear_fwd_rbias_add(y, ldy, x, ldx, scale_bias, d, (hipStream_t)stream);
    if (rc == RDB_E_UNSUPPORTED)
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_rbias_fwd: needs 16-byte aligned rows (pointers and leading dimensions) and fewer than "
                                            "2^29 elements per matrix");
    return rc;
}

extern "C" int rdb_linear_rbias_bwd(void *dx, int64_t lddx, float *d_scale_bias, const void *dy, int64_t lddy, const void *x, int64_t ldx,
                                    const void *scale_bias, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    int rc = check_desc("rdb_linear_rbias_bwd", d);
    if (rc) return rc;
    if (!dx || !dy || !scale_bias) return set_error(RDB_E_NULL, "rdb_linear_rbias_bwd: dx, dy or scale_bias is NULL");
    if (lddx < d->in_f || lddy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_rbias_bwd: leading dimension smaller than the row");
    if ((rc = rbias_request_ok("rdb_linear_rbias_bwd", d))) return rc;
    const char *why = "rdb_linear_rbias_bwd: needs 16-byte aligned rows (pointers and leading dimensions) and fewer than 2^29 elements per matrix";
    hipStream_t s = (hipStream_t)stream;
    if (!d_scale_bias) {
        rc = linear_dx_rbias_add(dx, lddx, dy, lddy, scale_bias, d, s);
        return rc == RDB_E_UNSUPPORTED ? set_error(RDB_E_UNSUPPORTED, "%s", why) : rc;
    }
    if (!x) return set_error(RDB_E_NULL, "rdb_linear_rbias_bwd: the gradient of the scale needs x");
    if (ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_rbias_bwd: leading dimension smaller than the row");
    const int64_t need = rdb_linear_workspace_bytes(RDB_OP_LINEAR_RBIAS_BWD, d);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3))
        return set_error(RDB_E_WORKSPACE, "rdb_linear_rbias_bwd: the gradient of the scale needs a workspace of %lld bytes", (long long)need);
    rc = linear_dx_rbias_add_dscale(dx, lddx, d_scale_bias, static_cast<float *>(workspace), dy, lddy, x, ldx, scale_bias, d, s);
    return rc == RDB_E_UNSUPPORTED ? set_error(RDB_E_UNSUPPORTED, "%s", why) : rc;
}

extern "C" int rdb_linear_bwd_dcoef(float *dcoef, float *d_scale_bias, const void *dy, int64_t lddy, const void *x, int64_t ldx,
                                    const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    int rc = check_desc("rdb_linear_bwd_dcoef", d);
    if (rc) return rc;
    const int64_t ncoef = (d->coef_rows ? d->coef_rows : 1) * d->k;
    if (ncoef > 0 && !dcoef) return set_error(RDB_E_NULL, "rdb_linear_bwd_dcoef: dcoef is NULL");
    hipStream_t s = (hipStream_t)stream;
    const bool empty = d->tokens == 0 || d->in_f == 0 || d->out_f == 0 || (ncoef == 0 && !d_scale_bias);
    if (!empty) {
        if (!dy || !x) return set_error(RDB_E_NULL, "rdb_linear_bwd_dcoef: dy or x is NULL");
        if (lddy < d->out_f || ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_bwd_dcoef: leading dimension smaller than the row");
    }
    if (!empty && d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16 && d->coef_rows != 0 && d->tokens <= 64 && !d_scale_bias) {
        // a few tokens: as in rdb_linear_fwd (dcoef is overwritten)
        rc = linear_dcoef_smallk(dcoef, dy, lddy, x, ldx, d, workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (!empty && d->algo == RDB_ALGO_AUTO && ncoef > 0 && vec_dcoef_two_pass_ok(d)) {
        // vector-coef with room for dW in the workspace: dW formed once (on the matrix cores at fp32 accuracy), then every element
        // of it contracted once with its k hashed values, at the rate of the hash (the general kernel below repeats the k hashes
        // per element for every block of tokens: 1.5 ms against 0.35 ms at 128 tokens x 768 -> 3072, k = 256)
        const int64_t need = vec_dcoef_workspace(d);
        if (need > 0 && workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0) {
            float *dW = static_cast<float *>(workspace);
            rc = linear_dw_f32(dW, dy, lddy, x, ldx, d, num_compute_units(), s);
            if (rc == RDB_OK) {
                const int64_t nw = d->out_f * d->in_f, mb = (rdb_materialize_bwd_workspace_bytes(0, d->k, 0, nw) + 255) / 256 * 256;
                char *after = static_cast<char *>(workspace) + linear_dw_f32_workspace(d, num_compute_units());
                rc = rdb_materialize_bwd(dcoef, dW, RDB_F32, 0, d->k, 0, nw, d->seed, after, mb, stream);
                if (rc == RDB_OK && d_scale_bias)
                    rc = rdb_scale_bias_bwd(d_scale_bias, dW, RDB_F32, nw, d->seed, after + mb, rdb_scale_bias_bwd_workspace_bytes(nw), stream);
                return rc;
            }
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
    }
    if (!empty && d->act_dtype == RDB_F32 && (d->algo == RDB_ALGO_AUTO || d->algo == RDB_ALGO_FACTORED)) {
        // The fp32 factored kernels overwrite their outputs: nothing to clear first.  The matrix-core kernels also return the
        // gradient of the random bias's scale.  Without it: the vector-ALU kernel's coefficient gradient grows with the tokens
        // (49 us at 256 tokens, 158 us at 1024 for 784 -> 512, k = 64; the matrix-core kernels take 39 us at 1028), so beyond
        // 128 tokens the matrix cores come first.
        const bool matrix_cores_first = d_scale_bias || d->tokens > 128;
        if (matrix_cores_first) {
            rc = linear_dcoef_f32(dcoef, d_scale_bias, dy, lddy, x, ldx, d, num_compute_units(), workspace, workspace_bytes, s);
            if (rc != RDB_E_UNSUPPORTED) return rc;
        }
        if (!d_scale_bias) {
            rc = linear_dcoef_smallk(dcoef, dy, lddy, x, ldx, d, workspace, workspace_bytes, s);
            if (rc != RDB_E_UNSUPPORTED) return rc;
            if (!matrix_cores_first) {
                rc = linear_dcoef_f32(dcoef, nullptr, dy, lddy, x, ldx, d, num_compute_units(), workspace, workspace_bytes, s);
                if (rc != RDB_E_UNSUPPORTED) return rc;
            }
        }
    }
    if (ncoef > 0) {
        rc = fill_zero(dcoef, ncoef, s);
        if (rc) return rc;
    }
    if (d_scale_bias) {
        rc = fill_zero(d_scale_bias, 1, s);
        if (rc) return rc;
    }
    if (empty) return RDB_OK;
    if ((d->algo == RDB_ALGO_AUTO || d->algo == RDB_ALGO_FACTORED) && !d_scale_bias) {
        rc = linear_dcoef_factored(dcoef, dy, lddy, x, ldx, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_FACTORED)
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dcoef: the factored algorithm needs matrix-coef, no scale_bias gradient, a "
                                            "workspace of rdb_linear_workspace_bytes() bytes and either bf16 activations (sizes that are "
                                            "multiples of 8; aligned rows) or fp32 (sizes that are multiples of 4; aligned rows)");
    if (d->algo != RDB_ALGO_TILE) {
        rc = linear_dcoef_fast(dcoef, d_scale_bias, dy, lddy, x, ldx, d, num_compute_units(), s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    if (d->algo == RDB_ALGO_AUTO && d->act_dtype == RDB_BF16) {
        // sizes that are not multiples of 8: the fp32 matrix cores, reading bf16 value by value (they overwrite what was cleared)
        rc = linear_dcoef_f32(dcoef, d_scale_bias, dy, lddy, x, ldx, d, num_compute_units(), workspace, workspace_bytes, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    const int es = d->act_dtype == RDB_BF16 ? 2 : 4;
    LinParams p = {};
    p.w = make_spec(d, nullptr, nullptr);
    p.a = dy;
    p.lda = lddy;
    p.b = x;
    p.ldb = ldx;
    p.dcoef = dcoef;
    p.dsb = d_scale_bias;
    p.tokens = d->tokens;
    p.vec_a = aligned16(dy) && (lddy * es) % 16 == 0;
    p.vec_b = aligned16(x) && (ldx * es) % 16 == 0;
    dim3 grid((unsigned)cdiv(d->in_f, BN), (unsigned)cdiv(d->out_f, BM));
    const bool mat = d->coef_rows != 0;
    if (d->act_dtype == RDB_BF16)
        return mat ? launch(linear_dcoef_kernel<bf16_t, true>, grid, smem_dcoef<bf16_t>(), s, p, "linear_dcoef_kernel<bf16,matrix>")
                   : launch(linear_dcoef_kernel<bf16_t, false>, grid, smem_dcoef<bf16_t>(), s, p, "linear_dcoef_kernel<bf16,vector>");
    return mat ? launch(linear_dcoef_kernel<float, true>, grid, smem_dcoef<float>(), s, p, "linear_dcoef_kernel<f32,matrix>")
               : launch(linear_dcoef_kernel<float, false>, grid, smem_dcoef<float>(), s, p, "linear_dcoef_kernel<f32,vector>");
}

// ----------------------------------------------------------------------------------------------- forward without a caller's workspace
// Scratch of rdb_linear_fwd_static: one copy per device that loads this library, held until the process ends.
#define RDB_STATIC_SCRATCH_BYTES (16ll << 20)
static __device__ __align__(256) unsigned char rdb_static_scratch[RDB_STATIC_SCRATCH_BYTES];

// Device address of the scratch array on the current device.  In host code the array's name is only a handle: the address
// is asked for once per device (with that device current) and kept.
static int static_scratch_ptr(void **out)
{
    static void *ptrs[64] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error((int)e, "rdb_linear_fwd_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd_static: device index %d outside 0..63", dev);
    void *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(rdb_static_scratch));
        if (e != hipSuccess || !p) return set_error(e != hipSuccess ? (int)e : RDB_E_UNSUPPORTED, "rdb_linear_fwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);   // every thread that gets here asks for the same address
    }
    *out = p;
    return RDB_OK;
}

extern "C" int64_t rdb_linear_fwd_static_max_bytes(void) { return RDB_STATIC_SCRATCH_BYTES; }

extern "C" int rdb_linear_fwd_static(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef, const void *scale_bias,
                                     const void *bias, const rdb_linear_desc *d, void *stream)
{
    int rc = check_desc("rdb_linear_fwd_static", d);
    if (rc) return rc;
    const int64_t need = rdb_linear_workspace_bytes(RDB_OP_LINEAR_FWD, d);
    if (need > RDB_STATIC_SCRATCH_BYTES)
        return set_error(RDB_E_WORKSPACE, "rdb_linear_fwd_static: this layer's kernels use %lld bytes of scratch, the library's static scratch holds "
                                          "%lld: call rdb_linear_fwd with a workspace of the caller's", (long long)need, (long long)RDB_STATIC_SCRATCH_BYTES);
    void *scratch = nullptr;
    if (need > 0) {
        rc = static_scratch_ptr(&scratch);
        if (rc) return rc;
    }
    return rdb_linear_fwd(y, ldy, x, ldx, coef, scale_bias, bias, d, scratch, need > 0 ? RDB_STATIC_SCRATCH_BYTES : 0, stream);
}

// ----------------------------------------------------------------------------------------------- projected entry points
// The kernels address activations with 32-bit byte offsets: one launch takes at most 2^29 elements of x, y, dy or dx.  Tokens
// are independent in y and dx and additive in dcoef, so a layer with more than that is run in chunks of tokens: every chunk
// is a layer of its own with its own projection state (the states lie one after the other in the caller's buffer), the
// chunks' dcoef are added up in chunk order (still the same bits from run to run), and one workspace serves them in turn.
struct ChunkPlan {
    int64_t chunk_tokens;  // tokens of every chunk but the last (a multiple of 256)
    int nchunks;           // 0: the projected form does not apply
    int64_t state_stride;  // bytes from one chunk's projection state to the next
};

static rdb_linear_desc chunk_desc(const rdb_linear_desc *d, const ChunkPlan &pl, int c)
{
    rdb_linear_desc dd = *d;
    const int64_t left = d->tokens - (int64_t)c * pl.chunk_tokens;
    dd.tokens = left < pl.chunk_tokens ? left : pl.chunk_tokens;
    return dd;
}

static ChunkPlan chunk_plan(const rdb_linear_desc *d)
{
    ChunkPlan pl = {0, 0, 0};
    if (!d || d->tokens <= 0 || d->in_f <= 0 || d->out_f <= 0 || d->k <= 0) return pl;
    const int64_t widest = std::max(std::max(d->in_f, d->out_f), cdiv(d->k, 64) * 64);
    // half the addressing limit, so that leading dimensions may exceed the row length by up to a factor of two
    int64_t per_chunk = ((1ll << 28) / widest) / 256 * 256;
    if (per_chunk < 256) return pl;
    int nchunks = (int)cdiv(d->tokens, per_chunk);
    if (nchunks > 1) per_chunk = cdiv(cdiv(d->tokens, nchunks), 256) * 256;   // chunks of about equal size
    else per_chunk = d->tokens;
    pl.chunk_tokens = per_chunk;
    pl.nchunks = (int)cdiv(d->tokens, per_chunk);
    const rdb_linear_desc first = chunk_desc(d, pl, 0);
    pl.state_stride = linear_projection_bytes(&first);
    if (pl.state_stride <= 0) pl.nchunks = 0;
    return pl;
}

static int check_projected(const char *who, const rdb_linear_desc *d, ChunkPlan *plan)
{
    int rc = check_desc(who, d);
    if (rc) return rc;
    const ChunkPlan pl = chunk_plan(d);
    if (pl.nchunks == 0)
        return set_error(RDB_E_UNSUPPORTED, "%s: the projected form needs matrix-coef, bf16 activations, non-empty sizes that are "
                                            "multiples of 8, and out_f*k (k rounded up to 64) below 2^29", who);
    if (plan) *plan = pl;
    return RDB_OK;
}

// fp32 layers: the state is z in fp32 (rdb_f32.hip), one chunk
static bool f32_projected(const rdb_linear_desc *d) { return d && d->act_dtype == RDB_F32; }
static int check_projected_f32(const char *who, const rdb_linear_desc *d)
{
    int rc = check_desc(who, d);
    if (rc) return rc;
    if (linear_f32_state_bytes(d) <= 0)
        return set_error(RDB_E_UNSUPPORTED, "%s: the projected form in fp32 needs matrix-coef, fp32 activations and coefficients, non-empty sizes "
                                            "and tokens * max(in_f, out_f) below 2^28", who);
    return RDB_OK;
}

extern "C" int64_t rdb_linear_projection_bytes(const rdb_linear_desc *d)
{
    if (f32_projected(d)) return check_desc("rdb_linear_projection_bytes", d) ? 0 : linear_f32_state_bytes(d);
    const ChunkPlan pl = chunk_plan(d);
    return pl.nchunks * pl.state_stride;
}

extern "C" int rdb_linear_projection_layout(const rdb_linear_desc *d, int64_t *info)
{
    if (f32_projected(d)) {   // z row-major in fp32 behind the header: info[1] = 0
        if (int rc = check_projected_f32("rdb_linear_projection_layout", d)) return rc;
        if (!info) return set_error(RDB_E_NULL, "rdb_linear_projection_layout: info is NULL");
        for (int i = 0; i < 8; ++i) info[i] = 0;
        info[0] = 256;
        info[4] = d->k;
        info[5] = d->tokens;
        return RDB_OK;
    }
    ChunkPlan pl;
    int rc = check_projected("rdb_linear_projection_layout", d, &pl);
    if (rc) return rc;
    if (!info) return set_error(RDB_E_NULL, "rdb_linear_projection_layout: info is NULL");
    if (pl.nchunks != 1) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_projection_layout: this layer's state is %d states of %lld tokens, one "
                                                            "after the other, %lld bytes apart: ask for the layout of one of them",
                                          pl.nchunks, (long long)pl.chunk_tokens, (long long)pl.state_stride);
    const ProjLayout L = proj_layout(d);
    info[0] = L.zf_off;
    info[1] = 1;
    info[2] = L.ztf_off;
    info[3] = L.ctf_off;
    info[4] = L.kpad;
    info[5] = L.tok32;
    info[6] = L.tok64;
    info[7] = L.out64;
    return RDB_OK;
}

// number of token chunks the projected entry points run `desc` in (1 for every layer whose activations fit one launch)
extern "C" int rdb_linear_projection_chunks(const rdb_linear_desc *d, int64_t *chunk_tokens)
{
    if (f32_projected(d)) {
        const bool ok = !check_desc("rdb_linear_projection_chunks", d) && linear_f32_state_bytes(d) > 0;
        if (chunk_tokens) *chunk_tokens = ok ? d->tokens : 0;
        return ok ? 1 : 0;
    }
    const ChunkPlan pl = chunk_plan(d);
    if (chunk_tokens) *chunk_tokens = pl.chunk_tokens;
    return pl.nchunks;
}

static char *at_bytes(const void *p, int64_t bytes) { return static_cast<char *>(const_cast<void *>(p)) + bytes; }

extern "C" int rdb_linear_project(void *state, const void *x, int64_t ldx, const void *coef, const rdb_linear_desc *d, void *stream)
{
    if (f32_projected(d)) {
        if (int rc = check_projected_f32("rdb_linear_project", d)) return rc;
        if (!state || !x) return set_error(RDB_E_NULL, "rdb_linear_project: state or x is NULL");
        if (ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_project: leading dimension smaller than the row");
        int rc = linear_project_f32(state, nullptr, 0, x, ldx, nullptr, nullptr, d, num_compute_units(), (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project: state must be 16-byte aligned and tokens * ldx below 2^29");
        return rc;
    }
    ChunkPlan pl;
    int rc = check_projected("rdb_linear_project", d, &pl);
    if (rc) return rc;
    if (!state || !x) return set_error(RDB_E_NULL, "rdb_linear_project: state or x is NULL");
    if (ldx < d->in_f) return set_error(RDB_E_SHAPE, "rdb_linear_project: leading dimension smaller than the row");
    if (coef && !aligned16(coef)) return set_error(RDB_E_ALIGN, "rdb_linear_project: coef must be 16-byte aligned");
    if (pl.chunk_tokens * ldx >= (1ll << 29) || ldx % 8 || !aligned16(x) || !aligned16(state))
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project: x and state must be 16-byte aligned, ldx a multiple of 8 and below twice in_f");
    for (int c = 0; c < pl.nchunks; ++c) {
        const rdb_linear_desc dd = chunk_desc(d, pl, c);
        rc = linear_project(at_bytes(state, c * pl.state_stride), at_bytes(x, c * pl.chunk_tokens * ldx * 2), ldx, coef, &dd, (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project: internal: chunk %d of %d refused", c, pl.nchunks);
        if (rc) return rc;
    }
    return RDB_OK;
}

extern "C" int rdb_linear_fwd_projected(void *y, int64_t ldy, const void *z, const void *coef, const void *bias, const rdb_linear_desc *d,
                                        void *stream)
{
    if (f32_projected(d)) {
        if (int rc = check_projected_f32("rdb_linear_fwd_projected", d)) return rc;
        if (!y || !z || !coef) return set_error(RDB_E_NULL, "rdb_linear_fwd_projected: y, z or coef is NULL");
        if (ldy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_fwd_projected: leading dimension smaller than the row");
        int rc = linear_fwd_projected_f32(y, ldy, z, coef, bias, d, num_compute_units(), (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd_projected: tokens * ldy must stay below 2^29");
        return rc;
    }
    ChunkPlan pl;
    int rc = check_projected("rdb_linear_fwd_projected", d, &pl);
    if (rc) return rc;
    if (!y || !z || !coef) return set_error(RDB_E_NULL, "rdb_linear_fwd_projected: y, z or coef is NULL");
    if (ldy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_fwd_projected: leading dimension smaller than the row");
    if (d->coef_dtype != RDB_BF16 || ldy % 8 || !aligned16(y) || !aligned16(z) || !aligned16(coef) || ((uintptr_t)bias & 7) ||
        pl.chunk_tokens * ldy >= (1ll << 29))
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd_projected: coefficients must be bf16; y, state and coef 16-byte aligned, bias 8-byte; "
                                            "ldy a multiple of 8 and below twice out_f");
    for (int c = 0; c < pl.nchunks; ++c) {
        const rdb_linear_desc dd = chunk_desc(d, pl, c);
        rc = linear_fwd_projected(at_bytes(y, c * pl.chunk_tokens * ldy * 2), ldy, at_bytes(z, c * pl.state_stride), coef, bias, &dd,
                                  num_compute_units(), (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_fwd_projected: internal: chunk %d of %d refused", c, pl.nchunks);
        if (rc) return rc;
    }
    return RDB_OK;
}

extern "C" int rdb_linear_project_fwd(void *y, int64_t ldy, void *state, const void *x, int64_t ldx, const void *coef, const void *bias,
                                      const rdb_linear_desc *d, void *stream)
{
    if (f32_projected(d)) {
        if (int rc = check_projected_f32("rdb_linear_project_fwd", d)) return rc;
        if (!y || !state || !x || !coef) return set_error(RDB_E_NULL, "rdb_linear_project_fwd: y, state, x or coef is NULL");
        if (ldx < d->in_f || ldy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_project_fwd: leading dimension smaller than the row");
        int rc = linear_project_f32(state, y, ldy, x, ldx, coef, bias, d, num_compute_units(), (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED)
            return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project_fwd: state must be 16-byte aligned and tokens * ldx, tokens * ldy below 2^29");
        return rc;
    }
    ChunkPlan pl;
    int rc = check_projected("rdb_linear_project_fwd", d, &pl);
    if (rc) return rc;
    if (!y || !state || !x || !coef) return set_error(RDB_E_NULL, "rdb_linear_project_fwd: y, state, x or coef is NULL");
    if (ldx < d->in_f || ldy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_project_fwd: leading dimension smaller than the row");
    if (d->coef_dtype != RDB_BF16 || ldx % 8 || ldy % 8 || !aligned16(x) || !aligned16(state) || !aligned16(y) || !aligned16(coef) ||
        ((uintptr_t)bias & 7) || pl.chunk_tokens * ldx >= (1ll << 29) || pl.chunk_tokens * ldy >= (1ll << 29))
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project_fwd: coefficients must be bf16; x, y, state and coef 16-byte aligned, bias 8-byte; "
                                            "leading dimensions multiples of 8 and below twice the row");
    for (int c = 0; c < pl.nchunks; ++c) {
        const rdb_linear_desc dd = chunk_desc(d, pl, c);
        rc = linear_project_fwd(at_bytes(y, c * pl.chunk_tokens * ldy * 2), ldy, at_bytes(state, c * pl.state_stride),
                                at_bytes(x, c * pl.chunk_tokens * ldx * 2), ldx, coef, true, bias, &dd, num_compute_units(), (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_project_fwd: internal: chunk %d of %d refused", c, pl.nchunks);
        if (rc) return rc;
    }
    return RDB_OK;
}

extern "C" int rdb_linear_bwd_dcoef_projected(float *dcoef, const void *dy, int64_t lddy, const void *z, const rdb_linear_desc *d, void *stream)
{
    if (f32_projected(d))
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dcoef_projected: fp32 sums over token ranges need scratch: call "
                                            "rdb_linear_bwd_projected with dx = NULL and a workspace");
    ChunkPlan pl;
    int rc = check_projected("rdb_linear_bwd_dcoef_projected", d, &pl);
    if (rc) return rc;
    if (!dcoef || !dy || !z) return set_error(RDB_E_NULL, "rdb_linear_bwd_dcoef_projected: dcoef, dy or z is NULL");
    if (lddy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_linear_bwd_dcoef_projected: leading dimension smaller than the row");
    if (lddy % 8 || !aligned16(dy) || !aligned16(z) || pl.chunk_tokens * lddy >= (1ll << 29))
        return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dcoef_projected: dy and z must be 16-byte aligned, lddy a multiple of 8 and below "
                                            "twice out_f");
    hipStream_t s = (hipStream_t)stream;
    if (pl.nchunks == 1 && big_bwd_applies(d, num_compute_units())) {
        // many 256 x 256 tiles of dcoef: each contracts all tokens and is stored once, nothing to clear or add
        rc = linear_bwd_big(nullptr, dcoef, dy, lddy, z, nullptr, d, num_compute_units(), false, true, s);
        if (rc != RDB_E_UNSUPPORTED) return rc;
    }
    rc = fill_zero(dcoef, d->coef_rows * d->k, s);
    if (rc) return rc;
    for (int c = 0; c < pl.nchunks; ++c) {   // every chunk adds its share with atomics
        const rdb_linear_desc dd = chunk_desc(d, pl, c);
        rc = linear_dcoef_projected(dcoef, at_bytes(dy, c * pl.chunk_tokens * lddy * 2), lddy, at_bytes(z, c * pl.state_stride), &dd, num_compute_units(), s);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_dcoef_projected: internal: chunk %d of %d refused", c, pl.nchunks);
        if (rc) return rc;
    }
    return RDB_OK;
}

// workspace of rdb_linear_bwd_projected: that of the largest chunk; chunks after the first add to dcoef and so always keep
// their sums in the workspace first
static int64_t bwd_projected_workspace(const rdb_linear_desc *d, bool force_partial)
{
    const ChunkPlan pl = chunk_plan(d);
    if (pl.nchunks == 0) return 0;
    const rdb_linear_desc first = chunk_desc(d, pl, 0);
    return linear_bwd_projected_workspace(&first, num_compute_units(), pl.nchunks > 1 || force_partial);
}

static int bwd_projected_entry(const char *who, void *dx, int64_t lddx, void *dcoef, int dcoef_dtype, const void *dy, int64_t lddy, const void *z,
                               const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (f32_projected(d)) {   // dx may be NULL: the coefficient gradient alone
        if (int rc = check_projected_f32(who, d)) return rc;
        if (!dcoef || !dy || !z || (dx && !coef)) return set_error(RDB_E_NULL, "%s: dcoef, dy, z or coef is NULL", who);
        if (lddy < d->out_f || (dx && lddx < d->in_f)) return set_error(RDB_E_SHAPE, "%s: leading dimension smaller than the row", who);
        if (dcoef_dtype != RDB_F32) return set_error(RDB_E_DTYPE, "%s: fp32 layers return dcoef in fp32", who);
        int rc = linear_bwd_projected_f32(dx, lddx, static_cast<float *>(dcoef), dy, lddy, z, coef, d, num_compute_units(), workspace, workspace_bytes,
                                          (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED)
            return set_error(RDB_E_UNSUPPORTED, "%s: needs a 16-byte aligned workspace of rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED) "
                                                "bytes and tokens * lddy, tokens * lddx below 2^29", who);
        return rc;
    }
    ChunkPlan pl;
    int rc = check_projected(who, d, &pl);
    if (rc) return rc;
    if (!dx || !dcoef || !dy || !z || !coef) return set_error(RDB_E_NULL, "%s: dx, dcoef, dy, z or coef is NULL", who);
    if (lddy < d->out_f || lddx < d->in_f) return set_error(RDB_E_SHAPE, "%s: leading dimension smaller than the row", who);
    if (dcoef_dtype != RDB_F32 && dcoef_dtype != RDB_BF16) return set_error(RDB_E_DTYPE, "%s: dcoef_dtype must be RDB_F32 or RDB_BF16", who);
    const bool dc_bf16 = dcoef_dtype == RDB_BF16;
    const rdb_linear_desc first = chunk_desc(d, pl, 0);
    if (d->coef_dtype != RDB_BF16 || lddy % 8 || lddx % 8 || !aligned16(dy) || !aligned16(dx) || !aligned16(z) || !aligned16(coef) ||
        !aligned16(dcoef) || !aligned16(workspace) || pl.chunk_tokens * lddy >= (1ll << 29) || pl.chunk_tokens * lddx >= (1ll << 29) || !workspace ||
        workspace_bytes < linear_dx_factored_workspace(&first))
        return set_error(RDB_E_UNSUPPORTED, "%s: coefficients must be bf16; all pointers 16-byte aligned; lddy, lddx multiples of 8 and below "
                                            "twice the row; workspace of rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX) bytes at least", who);
    if (dc_bf16 && (pl.nchunks > 1 || workspace_bytes < bwd_projected_workspace(d, true)))
        return set_error(RDB_E_UNSUPPORTED, "%s: dcoef in bf16 needs a layer that runs as one chunk of tokens and a workspace of "
                                            "rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED_TO) bytes", who);
    for (int c = 0; c < pl.nchunks; ++c) {
        const rdb_linear_desc dd = chunk_desc(d, pl, c);
        rc = linear_bwd_projected(at_bytes(dx, c * pl.chunk_tokens * lddx * 2), lddx, static_cast<float *>(dcoef),
                                  at_bytes(dy, c * pl.chunk_tokens * lddy * 2), lddy, at_bytes(z, c * pl.state_stride), coef, &dd,
                                  num_compute_units(), workspace, workspace_bytes, c > 0, dc_bf16, (hipStream_t)stream);
        if (rc == RDB_E_UNSUPPORTED) return set_error(RDB_E_UNSUPPORTED, "%s: internal: chunk %d of %d refused", who, c, pl.nchunks);
        if (rc) return rc;
    }
    return RDB_OK;
}

extern "C" int rdb_linear_bwd_projected(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *z, const void *coef,
                                        const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    return bwd_projected_entry("rdb_linear_bwd_projected", dx, lddx, dcoef, RDB_F32, dy, lddy, z, coef, d, workspace, workspace_bytes, stream);
}

namespace rdb {
void set_bwd_projected_parts(int mask);   // rdb_dx.hip
}

extern "C" int rdb_linear_bwd_projected_part(int part, void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *z,
                                             const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (part != 1 && part != 2) return set_error(RDB_E_SHAPE, "rdb_linear_bwd_projected_part: part must be 1 or 2");
    if (d && d->act_dtype != RDB_BF16) return set_error(RDB_E_UNSUPPORTED, "rdb_linear_bwd_projected_part: bf16 layers only");
    if (d && workspace_bytes < bwd_projected_workspace(d, false))
        return set_error(RDB_E_WORKSPACE, "rdb_linear_bwd_projected_part: needs the workspace of rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED)");
    set_bwd_projected_parts(part);
    const int rc = bwd_projected_entry("rdb_linear_bwd_projected_part", dx, lddx, dcoef, RDB_F32, dy, lddy, z, coef, d, workspace, workspace_bytes, stream);
    set_bwd_projected_parts(3);
    return rc;
}

extern "C" int rdb_linear_bwd_projected_to(void *dx, int64_t lddx, void *dcoef, int dcoef_dtype, const void *dy, int64_t lddy, const void *z,
                                           const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, void *stream)
{
    return bwd_projected_entry("rdb_linear_bwd_projected_to", dx, lddx, dcoef, dcoef_dtype, dy, lddy, z, coef, d, workspace, workspace_bytes, stream);
}

// rdb_factored.hip, rdb_smallk.hip
namespace rdb {
int selftest_giveup_factored(void *y, int64_t ldy, void *state, const void *coef, const rdb_linear_desc *d, int num_cus, int polls, hipStream_t s);
int selftest_giveup_smallk(void *y, int64_t ldy, const void *coef, const rdb_linear_desc *d, void *workspace, int64_t workspace_bytes, int polls,
                           hipStream_t s);
}

extern "C" int rdb_selftest_sync_giveup(void *y, int64_t ldy, void *scratch, int64_t scratch_bytes, const void *coef, const rdb_linear_desc *d,
                                        int polls, void *stream)
{
    int rc = check_desc("rdb_selftest_sync_giveup", d);
    if (rc) return rc;
    if (!y || !scratch || !coef) return set_error(RDB_E_NULL, "rdb_selftest_sync_giveup: y, scratch or coef is NULL");
    if (polls < 1 || polls > SYNC_SPIN_LIMIT) return set_error(RDB_E_SHAPE, "rdb_selftest_sync_giveup: polls must be 1 .. %d", SYNC_SPIN_LIMIT);
    if (ldy < d->out_f) return set_error(RDB_E_SHAPE, "rdb_selftest_sync_giveup: leading dimension smaller than the row");
    if (d->act_dtype == RDB_BF16) {
        const ChunkPlan pl = chunk_plan(d);
        if (pl.nchunks != 1 || scratch_bytes < pl.state_stride) rc = RDB_E_UNSUPPORTED;
        else rc = selftest_giveup_factored(y, ldy, scratch, coef, d, num_compute_units(), polls, (hipStream_t)stream);
    } else {
        rc = selftest_giveup_smallk(y, ldy, coef, d, scratch, scratch_bytes, polls, (hipStream_t)stream);
    }
    if (rc == RDB_E_UNSUPPORTED)
        return set_error(RDB_E_UNSUPPORTED, "rdb_selftest_sync_giveup: needs a layer whose forward has a one-launch form (bf16 matrix-coef, k <= 256, "
                                            "or fp32 matrix-coef, k <= 64, in_f <= 8192) and its scratch (projection state / forward workspace)");
    return rc;
}

namespace rdb {
int set_f32_split_mode(int mode);   // rdb_f32.hip
}
extern "C" int rdb_set_f32_split(int mode) { return rdb::set_f32_split_mode(mode); }

extern "C" int rdb_set_big_tiles(int mode)
{
    const int before = big_tiles_mode();
    set_big_tiles_mode(mode);
    return before;
}
