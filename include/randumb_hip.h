/*
 * randumb_hip.h - C ABI of librandumb_hip.so, the gfx950 (MI355X) implementation of RANDUMB's
 * pseudorandom-matrix hot path.
 *
 * A pseudorandom tensor is  W = Noise(seed) . coef : the noise is Squirrel5 integer-hash noise in
 * [-1, 1] addressed by (seed, index) and is never stored; only coef is trainable.
 *
 * Conventions shared by every entry point
 *   - all pointers are DEVICE pointers on the current HIP device unless stated otherwise;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work is enqueued, not awaited;
 *   - nothing is allocated or freed inside the library; outputs and workspaces belong to the caller;
 *   - return value: 0 = ok, < 0 = argument error (RDB_E_*), > 0 = a hipError_t from a launch;
 *     rdb_last_error_string() describes the last non-zero return on the calling thread;
 *   - dtype codes: RDB_F32 = 0, RDB_BF16 = 1 (rdb_dtype);
 *   - seeds are uint32 (the reference is exercised with 0 <= seed < 2^31);
 *   - "vector-coef" = the reference form, one coef vector c[k] for the whole tensor:
 *         W_flat[a] = sum_m noise(PRIME*a + m) * c[m],  a = storage offset of the element;
 *     "matrix-coef" = the row-batched form, coef C[rows x k] over a contiguous (rows, row_len) tensor:
 *         W[o, i] = sum_m noise(PRIME*i + m) * C[o, m]
 *     (row o alone is a vector-coef tensor of shape (row_len,) with coef C[o, :]).
 *
 * Reference citations are to Clyde013/randumb, paths relative to its checkout:
 *   R.py  = src/rten_cpp/RandumbTensor.py      R.cu = src/rten_cpp/csrc/cuda/rten.cu
 *   R.cpp = src/rten_cpp/csrc/rten.cpp
 */
#ifndef RANDUMB_HIP_H
#define RANDUMB_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { RDB_F32 = 0, RDB_BF16 = 1 } rdb_dtype;

enum {
    RDB_OK = 0,
    RDB_E_NULL = -1,        /* a required pointer is NULL */
    RDB_E_SHAPE = -2,       /* a size is negative, zero where it must not be, or too large */
    RDB_E_DTYPE = -3,       /* unknown or unsupported dtype code / combination */
    RDB_E_ALIGN = -4,       /* pointer or leading dimension not aligned as required */
    RDB_E_UNSUPPORTED = -5, /* valid request this build has no kernel for */
    RDB_E_WORKSPACE = -6    /* workspace missing or too small */
};

/* Library identification; bumps when an entry point changes meaning. */
int rdb_abi_version(void);

/* Text for the last non-zero return code on this thread (never NULL). */
const char *rdb_last_error_string(void);

/* ------------------------------------------------------------------------------------------ noise probes
 * Replace: squirrel5_generate_2d / squirrel5_kernel_2d (R.py:78-105), rten_cpp::sq5_gen_2d (R.cpp:37,
 * R.cu:50-71; its store index bug for non-square shapes is not reproduced).
 * out is fp32 [N x M] row-major, out[n*M + m] = noise(PRIME*n + m, seed). */
int rdb_sq5_fill_2d(float *out, int64_t N, int64_t M, uint32_t seed, void *stream);

/* Replace: squirrel5_generate_1d / squirrel5_kernel_1d (R.py:108-126).  out[n] = noise(n, seed). */
int rdb_sq5_fill_1d(float *out, int64_t N, uint32_t seed, void *stream);

/* ------------------------------------------------------------------------------------------ materialise
 * Replaces: op rten::materialize_fwd + materialize_fwd_kernel (R.py:235-290, 371-381) and
 * rten_cpp::materialize_fwd (R.cpp:38, R.cu:74-152).
 * Writes the (P, Q) view with element strides (sP, sQ) of the pseudorandom tensor, contiguous fp32:
 *     out[p*Q + q] = W_flat[a],  a = q*sQ + p*sP                                   (R.py:264)
 * coef_rows == 0: vector-coef, coef is [k].  coef_rows > 0: matrix-coef, coef is [coef_rows x k]
 * contiguous and `a` addresses a contiguous (coef_rows, row_len) tensor.
 * scale_bias: NULL, or a device pointer to ONE value of dtype coef_dtype; adds
 *     scale_bias[0] * noise(a, seed)  (the fused random bias, R.py:286-289).
 * A 1-D tensor of Q elements is passed as P = 1, sP = 0 (R.py:375-377). */
int rdb_materialize_fwd(float *out, const void *coef, int coef_dtype, int64_t coef_rows, int64_t k,
                        int64_t row_len, int64_t P, int64_t Q, int64_t sP, int64_t sQ, uint32_t seed,
                        const void *scale_bias, void *stream);

/* Replaces: op rten::materialize_bwd + materialize_bwd_kernel (R.py:304-359, 383-390).
 * dW is a contiguous tensor of Nw elements (dtype dw_dtype).  dcoef is fp32 and is OVERWRITTEN:
 *   vector-coef (coef_rows == 0): dcoef[m] = sum_a noise(PRIME*a + m) * dW[a],              dcoef is [k]
 *   matrix-coef: Nw = coef_rows*row_len, dcoef[o*k+m] = sum_i noise(PRIME*i + m) * dW[o*row_len+i].
 * The reduction is a fixed tree (no atomics): results are bitwise reproducible run to run.
 * workspace: device scratch of at least rdb_materialize_bwd_workspace_bytes(...) bytes (may be NULL
 * when that returns 0).  Matrix-coef tensors of some millions of multiply-adds or more run as the matrix
 * product dW . N^T on the fp32 matrix cores with the noise hashed as an operand (rdb_materialize_fwd: C . N
 * likewise); the workspace then holds the sums over ranges of the row, added up in range order; with less
 * workspace than the query asks for the vector-ALU kernel runs instead. */
int rdb_materialize_bwd(float *dcoef, const void *dW, int dw_dtype, int64_t coef_rows, int64_t k,
                        int64_t row_len, int64_t Nw, uint32_t seed, void *workspace,
                        int64_t workspace_bytes, void *stream);
int64_t rdb_materialize_bwd_workspace_bytes(int64_t coef_rows, int64_t k, int64_t row_len, int64_t Nw);

/* Replaces: op rten::scale_bias_bwd + scale_bias_bwd_kernel (R.py:399-420).
 * ds[0] = sum_a dW[a] * noise(a, seed) over the contiguous dW; fp32, overwritten, deterministic.
 * workspace: at least rdb_scale_bias_bwd_workspace_bytes(Nw) bytes. */
int rdb_scale_bias_bwd(float *ds, const void *dW, int dw_dtype, int64_t Nw, uint32_t seed,
                       void *workspace, int64_t workspace_bytes, void *stream);
int64_t rdb_scale_bias_bwd_workspace_bytes(int64_t Nw);

/* ------------------------------------------------------------------------------------------ embedding
 * Replaces: op rten::embed_fwd + embed_fwd_kernel (R.py:998-1057, 1121-1126).
 * out[j*rowsize + r] = sum_m noise(PRIME*(idx[j]*rowsize + r) + m) * coef[m];  out fp32 [n_idx x rowsize],
 * idx int64 [n_idx], coef vector-coef [k]. */
int rdb_embed_fwd(float *out, const int64_t *idx, int64_t n_idx, const void *coef, int coef_dtype,
                  int64_t k, int64_t rowsize, uint32_t seed, void *stream);

/* Replaces: op rten::embed_bwd + embed_bwd_kernel (R.py:1059-1108, 1128-1134).
 * dcoef[m] = sum_{j,r} noise(PRIME*(idx[j]*rowsize + r) + m) * dout[j*rowsize + r]; fp32 [k], overwritten,
 * deterministic.  workspace: at least rdb_embed_bwd_workspace_bytes(n_idx, rowsize, k) bytes. */
int rdb_embed_bwd(float *dcoef, const int64_t *idx, int64_t n_idx, const void *dout, int dout_dtype,
                  int64_t k, int64_t rowsize, uint32_t seed, void *workspace, int64_t workspace_bytes,
                  void *stream);
int64_t rdb_embed_bwd_workspace_bytes(int64_t n_idx, int64_t rowsize, int64_t k);

/* ------------------------------------------------------------------------------------------ fused linear
 * The pseudorandom weight W is (out_f, in_f); element (o, i) has storage offset a = o*sO + i*sI
 * (F.linear's weight: sO = in_f, sI = 1; `mat1 @ tensor` with a contiguous (P, Q) tensor: out_f = Q,
 * in_f = P, sO = 1, sI = Q).  W is regenerated tile by tile on chip and never written to memory.
 * coef_rows == 0: vector-coef, coef [k];  coef_rows == out_f: matrix-coef, coef [out_f x k] (requires
 * sO = in_f, sI = 1; the noise row is i).
 * scale_bias: NULL or one device value of coef_dtype: W += scale_bias[0]*noise(a).
 * act_dtype is the dtype of x / y / dy / dx: RDB_BF16 computes with bf16 MFMA and fp32 accumulation
 * (W rounded to bf16 once, after its fp32 accumulation, as materialize().to(dtype) does, R.py:892);
 * RDB_F32 computes with fp32 MFMA.  Leading dimensions are in elements.
 */
typedef struct rdb_linear_desc {
    int64_t tokens;     /* rows of x / y / dy / dx */
    int64_t in_f;       /* W columns, contraction dim of the forward */
    int64_t out_f;      /* W rows */
    int64_t k;          /* coef length */
    int64_t coef_rows;  /* 0 = vector-coef, out_f = matrix-coef */
    int64_t sO, sI;     /* storage strides of W's (o, i) element */
    uint32_t seed;
    int32_t act_dtype;  /* rdb_dtype of activations and their gradients */
    int32_t coef_dtype; /* rdb_dtype of coef and scale_bias */
    int32_t algo;       /* RDB_ALGO_* ; 0 = let the library choose */
} rdb_linear_desc;

enum {
    RDB_ALGO_AUTO = 0, /* fastest kernel the request qualifies for */
    RDB_ALGO_TILE = 1, /* regenerate W blocks in LDS per output block, contract with MFMA (any shape/dtype) */
    RDB_ALGO_STRIP = 2, /* form W on chip with the noise hashed once per workgroup (matrix-coef, bf16 activations).
                           forward: a whole strip W[strip, 0:in] is built in LDS, then the tokens stream through it (the
                           strip must fit LDS).  dx: the workgroup keeps the noise columns of its 128 input features in
                           LDS and re-forms W in chunks of 64 output rows on the matrix cores (bf16 coef, k <= 256, no
                           scale_bias).  dcoef: dW tiles are formed and contracted with regenerated noise on chip. */
    RDB_ALGO_FACTORED = 3 /* matrix-coef only: use W = C.N associatively so that no weight tile is formed:
                             y = (x.N^T).C^T, dx = (dy.C).N, dcoef = dy^T.(x.N^T); the [tokens x k] intermediate lives in
                             the caller's workspace.  bf16 activations and coef (sizes multiples of 8): bf16 matrix cores;
                             fp32, or bf16 with other sizes: fp32 matrix cores; a few tokens (k <= 64 in fp32 up to 1024
                             tokens; under AUTO also k <= 256 up to 96 tokens in either dtype): the vector ALU, in fp32;
                             partial sums are added in a fixed order.  With scale_bias the full-rank share s.R is
                             one more product with R hashed as an operand. */
};

enum { RDB_OP_LINEAR_FWD = 0, RDB_OP_LINEAR_BWD_DX = 1, RDB_OP_LINEAR_BWD_DCOEF = 2, RDB_OP_LINEAR_BWD_PROJECTED = 3,
       RDB_OP_LINEAR_BWD_PROJECTED_TO = 4, RDB_OP_LINEAR_BWD_DX_DSCALE = 5, RDB_OP_LINEAR_RBIAS_BWD = 6 };

/* Device scratch (bytes) that entry point `op` can use for `desc`; 0 when it has no use for any.  A NULL or too small
 * workspace is never an error with RDB_ALGO_AUTO: the library then runs a kernel that needs none. */
int64_t rdb_linear_workspace_bytes(int op, const rdb_linear_desc *desc);

/* Replaces the dispatch of aten.mm / aten.addmm on a pseudorandom tensor: materialize() then the dense
 * product fakeMM (R.py:771-791, 942-952), and the experimental rt_mm (R.py:457-645).
 * y[t, o] = sum_i x[t, i] * W[o, i]  (+ bias[o] if bias != NULL; bias has act_dtype). */
int rdb_linear_fwd(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef,
                   const void *scale_bias, const void *bias, const rdb_linear_desc *desc, void *workspace,
                   int64_t workspace_bytes, void *stream);

/* rdb_linear_fwd for callers that can neither allocate a workspace nor hand one over (code under HIP graph capture, tight
 * serving loops, harnesses that forbid allocation); it has no counterpart in the reference.  Same arguments and results as
 * rdb_linear_fwd without the workspace: the scratch its kernels use (the projection of x) lies in a static device array of
 * the library, rdb_linear_fwd_static_max_bytes() = 16 MiB per device.  A layer whose kernels would use more returns
 * RDB_E_WORKSPACE and launches nothing (8192 tokens at k = 256, out_f = 3072 use 9.5 MiB).  The call allocates and frees
 * nothing.  All calls on one device share the array: calls that overlap in time on one device (different streams or
 * threads) race; on one stream they are ordered.  Nothing in the array has to be cleared between calls. */
int rdb_linear_fwd_static(void *y, int64_t ldy, const void *x, int64_t ldx, const void *coef,
                          const void *scale_bias, const void *bias, const rdb_linear_desc *desc, void *stream);
int64_t rdb_linear_fwd_static_max_bytes(void);

/* Replaces autograd's MmBackward on the materialised weight (second materialize() + dense product).
 * dx[t, i] = sum_o dy[t, o] * W[o, i]. */
int rdb_linear_bwd_dx(void *dx, int64_t lddx, const void *dy, int64_t lddy, const void *coef,
                      const void *scale_bias, const rdb_linear_desc *desc, void *workspace,
                      int64_t workspace_bytes, void *stream);

/* rdb_linear_bwd_dx for a layer with the fused random bias (W = C.N + s.R), and on the side the gradient of s:
 *   dx[t, i] = sum_o dy[t, o] * W[o, i]        d_scale_bias[0] = sum_{o,i} (dy^T x)[o, i] * R[o, i] = <dy . R, x>   (fp32, overwritten)
 * The random-bias share dy . R is a full-rank product that the input gradient forms anyway; reducing it against x in the same
 * pass gives what scale_bias_bwd computes from a stored dW (R.py:399-420, 988), so that the coefficient gradient can come from
 * rdb_linear_bwd_dcoef without d_scale_bias, i.e. from the factored kernels, and dW is never formed.  Partial sums are added in a
 * fixed order.  Needs matrix-coef, bf16 activations and coefficients, sizes that are multiples of 8, a workspace of
 * rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX_DSCALE, desc) bytes; otherwise RDB_E_UNSUPPORTED and nothing is launched. */
int rdb_linear_bwd_dx_dscale(void *dx, int64_t lddx, float *d_scale_bias, const void *dy, int64_t lddy, const void *x,
                             int64_t ldx, const void *coef, const void *scale_bias, const rdb_linear_desc *desc,
                             void *workspace, int64_t workspace_bytes, void *stream);

/* The random-bias share of a layer with W = C.N + s.R (R[o, i] = noise1d(o*in_f + i), the term materialize adds at
 * R.py:286-289) on its own, ADDED to a matrix that already holds the low-rank share; for callers that run that share through
 * the projected entry points below (projection state saved by the forward pass, so that the backward pass forms x.N^T only
 * once).  desc->k and the coefficients play no part.
 *   rdb_linear_rbias_fwd:  y[t, o]  += s * sum_i x[t, i]  * R[o, i]
 *   rdb_linear_rbias_bwd:  dx[t, i] += s * sum_o dy[t, o] * R[o, i];  when d_scale_bias != NULL also
 *                          d_scale_bias[0] = <dy . R, x> (fp32, overwritten; what scale_bias_bwd computes from a stored dW,
 *                          R.py:399-420), from the same pass; x and a workspace of
 *                          rdb_linear_workspace_bytes(RDB_OP_LINEAR_RBIAS_BWD, desc) bytes are needed then only.
 * bf16 activations and scale (one bf16 value), matrix-coef descriptor, sizes that are multiples of 8, 16-byte aligned rows;
 * RDB_E_UNSUPPORTED and nothing launched otherwise.  Sums in a fixed order: the same bits from run to run. */
int rdb_linear_rbias_fwd(void *y, int64_t ldy, const void *x, int64_t ldx, const void *scale_bias,
                         const rdb_linear_desc *desc, void *stream);
int rdb_linear_rbias_bwd(void *dx, int64_t lddx, float *d_scale_bias, const void *dy, int64_t lddy, const void *x,
                         int64_t ldx, const void *scale_bias, const rdb_linear_desc *desc, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* Replaces MmBackward's dW = dy^T x followed by RandumbTensorConstructor.backward ->
 * materialize_bwd (+ scale_bias_bwd) (R.py:979-990): dW is contracted with the regenerated noise tile
 * as it is produced and never written to memory.  (One exception, the reference's own data flow: a vector-coef layer whose
 * weight is contiguous, under RDB_ALGO_AUTO with the workspace rdb_linear_workspace_bytes asks for, forms dW in fp32 in that
 * workspace once and contracts it once, every element with its k hashed values, at the rate of the hash; without the
 * workspace the general kernel repeats those k hashes per element for every block of tokens.  Sums in a fixed order.)
 * dcoef (fp32, [k] or [out_f x k]) and, when d_scale_bias != NULL, d_scale_bias (fp32 [1]) are
 * OVERWRITTEN.  fp32 activations: partial sums are added in a fixed order, the result is the same bit for
 * bit from run to run.  bf16 activations: partial sums from different tiles are combined with fp32 atomics
 * (order-dependent in the last bits, like the reference's relaxed atomics, R.py:359);
 * rdb_linear_bwd_projected is the bf16 entry point with ordered sums. */
int rdb_linear_bwd_dcoef(float *dcoef, float *d_scale_bias, const void *dy, int64_t lddy, const void *x,
                         int64_t ldx, const rdb_linear_desc *desc, void *workspace, int64_t workspace_bytes,
                         void *stream);

/* -------------------------------------------------------------------------- fused linear, projected form
 * For matrix-coef layers with bf16 activations, z = x . N^T ([tokens x k], bf16: the activations projected onto the k
 * noise directions of this layer's weight) is all that the forward product and the coefficient gradient need of x:
 *   y = z . C^T (+ bias)        dcoef = dy^T . z
 * rdb_linear_fwd and rdb_linear_bwd_dcoef compute z into their workspace on every call.  A training step can instead
 * compute it once, keep it from the forward to the backward pass (the backward pass then needs nothing else of x; whether x
 * itself can be freed depends on who else holds it) and call the consumers below.  fp32 layers likewise, with z in fp32.  Replaces,
 * like rdb_linear_fwd / rdb_linear_bwd_dcoef, materialize() + dense product (R.py:942-952) and MmBackward's dW followed by
 * materialize_bwd (R.py:979-990, 304-359); the tensor autograd saves for the backward pass (there: x, with W
 * re-materialised) becomes the projection state.
 *
 * The projection STATE is an opaque caller-owned device buffer of rdb_linear_projection_bytes(desc) bytes, 16-byte aligned,
 * written by rdb_linear_project and read by the other three.  It holds z in the element orders its consumers' matrix
 * instructions take their operands in (z for the forward product, z transposed for the coefficient gradient; about
 * 2 * tokens * k * 2 bytes with k rounded up to 64) and, if rdb_linear_project was given the coefficients, C transposed for
 * the input gradient (out_f * k * 2 bytes): the kernels then fetch these small operands straight into registers and only
 * the large operand (dy) is staged through on-chip memory.  Needs: coef_rows == out_f, act_dtype RDB_BF16,
 * tokens/in_f/out_f/k > 0, in_f, out_f, k multiples of 8, out_f*k (k and out_f rounded up to 64) below 2^29, 16-byte
 * aligned pointers, leading dimensions multiples of 8; otherwise RDB_E_UNSUPPORTED. */

/* Bytes of the projection state for `desc`, or 0 when the projected form does not apply to it. */
int64_t rdb_linear_projection_bytes(const rdb_linear_desc *desc);

/* One launch addresses at most 2^29 elements of x, y, dy or dx.  The projected entry points take any number of tokens all
 * the same: tokens are independent in y and dx and additive in dcoef, so a layer with more is run in chunks of tokens (a
 * multiple of 256 each), every chunk with a projection state of its own, one after the other in the state buffer; dcoef is
 * added up in chunk order (the same bits from run to run) and one workspace serves the chunks in turn.  The reference has
 * no such limit and no counterpart of this (R.py:942-946 is one dense product).  Returns the number of chunks (1 for every
 * layer whose activations fit one launch, 0 when the projected form does not apply) and, if chunk_tokens != NULL, the tokens
 * per chunk (the last chunk may hold fewer).  Leading dimensions may exceed the row length by up to a factor of two. */
int rdb_linear_projection_chunks(const rdb_linear_desc *desc, int64_t *chunk_tokens);

/* Where the pieces lie inside the state, for tools and tests that want to look at z (no reference counterpart: the
 * reference keeps x).  Returns 0 and fills info[0..7], or RDB_E_UNSUPPORTED:
 *   info[0] byte offset of z for the forward product    info[1] 1 (fragment order, rows = tokens)
 *   info[2] byte offset of z transposed (fragment order, rows = coefficients)
 *   info[3] byte offset of C transposed (fragment order, rows = coefficients); valid when the state's first 32-bit word is 1
 *   info[4] k rounded up to 64   info[5] tokens rounded up to 32   info[6] tokens rounded up to 64   info[7] out_f rounded up to 64
 * Fragment order of a matrix M[row][kk] with `ksteps` = (padded kk extent) / 16 k-steps per block of 32 rows:
 *   element (row, kk) at ((row/32)*ksteps + kk/16)*512 + ((kk/8)%2*32 + row%32)*8 + kk%8   (in elements). */
int rdb_linear_projection_layout(const rdb_linear_desc *desc, int64_t *info);

/* state <- z[t, m] = sum_i x[t, i] * noise(PRIME*i + m), rounded to bf16 once.  coef: NULL, or the layer's bf16
 * coefficients [out_f x k], whose transposed copy then goes into the state for rdb_linear_bwd_projected; the values the
 * backward pass is later given as `coef` must be the same (as they are between the forward and the backward pass of one
 * training step).  A state written with coef == NULL serves every consumer too (rdb_linear_bwd_projected then reads the
 * coefficients through on-chip memory). */
int rdb_linear_project(void *state, const void *x, int64_t ldx, const void *coef, const rdb_linear_desc *desc,
                       void *stream);

/* rdb_linear_project (with coef) and rdb_linear_fwd_projected in one call: state <- projection of x and transposed coef,
 * y[t, o] = sum_m z[t, m] * coef[o, m] (+ bias[o]); coef must be bf16.  The forward pass of a training step (R.py:942-946
 * with what autograd saves replaced by the state).  With k <= 256 it is a single kernel launch: the blocks that multiply
 * start as the blocks that project leave the compute units, each waiting only for the 256 tokens it reads (per-tile tags
 * inside the state, unique to the launch; the hardware hands out a launch's blocks in index order, so the waiting blocks
 * cannot starve the ones they wait for; the wait is bounded and a block that gives up sets the state's second 32-bit word,
 * which no run has shown).  Results are bit for bit those of the two separate calls. */
int rdb_linear_project_fwd(void *y, int64_t ldy, void *state, const void *x, int64_t ldx, const void *coef,
                           const void *bias, const rdb_linear_desc *desc, void *stream);

/* y[t, o] = sum_m z[t, m] * coef[o, m] (+ bias[o]); coef must be bf16. */
int rdb_linear_fwd_projected(void *y, int64_t ldy, const void *state, const void *coef, const void *bias,
                             const rdb_linear_desc *desc, void *stream);

/* dcoef[o, m] = sum_t dy[t, o] * z[t, m]; fp32 [out_f x k], OVERWRITTEN; partial sums over token ranges are combined
 * with fp32 atomics. */
int rdb_linear_bwd_dcoef_projected(float *dcoef, const void *dy, int64_t lddy, const void *state,
                                   const rdb_linear_desc *desc, void *stream);

/* Whole backward pass of the layer from the projection state, in two kernel launches instead of five:
 * dx[t, i] = sum_o dy[t, o] * W[o, i] (act dtype) and dcoef = dy^T . z (fp32, OVERWRITTEN).
 * workspace: rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED, desc) bytes holds dy.C and the partial sums of dcoef
 * over token ranges.  Then the first launch runs the two long contractions over dy (dy.C and the dcoef partial sums) side by
 * side, and the second the (dy.C).N blocks beside blocks that add the partial sums in a fixed order: no atomics, the
 * result is the same bit for bit from run to run.  With the RDB_OP_LINEAR_BWD_DX amount only (room for dy.C) the first
 * launch computes dy.C and clears dcoef, and the second combines the dcoef blocks with fp32 atomics beside (dy.C).N.
 * Same requirements as the other projected entry points, coef in bf16; dcoef 16-byte aligned. */
int rdb_linear_bwd_projected(void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy, const void *state,
                             const void *coef, const rdb_linear_desc *desc, void *workspace,
                             int64_t workspace_bytes, void *stream);

/* rdb_linear_bwd_projected with dcoef in the dtype the caller keeps its coefficients in: dcoef_dtype RDB_F32 (the call above)
 * or RDB_BF16, [out_f x k], the fp32 sums rounded to bf16 once by the blocks that add them up; what
 * RandumbTensorConstructor.backward does with `.to(ctx.dtype)` after materialize_bwd (R.py:986), without the extra pass over
 * dcoef.  RDB_BF16 needs a workspace of rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED_TO, desc) bytes and a layer
 * that runs as one chunk of tokens (rdb_linear_projection_chunks == 1); otherwise RDB_E_UNSUPPORTED and nothing is launched. */
int rdb_linear_bwd_projected_to(void *dx, int64_t lddx, void *dcoef, int dcoef_dtype, const void *dy, int64_t lddy,
                                const void *state, const void *coef, const rdb_linear_desc *desc, void *workspace,
                                int64_t workspace_bytes, void *stream);

/* For tools that time the two kernel launches of rdb_linear_bwd_projected one by one (no counterpart in the reference):
 * part 1 enqueues only the first launch (dy.C into the workspace and the partial sums of dcoef), part 2 only the second
 * ((dy.C).N into dx and the ordered sum into dcoef, from what a first launch left in the workspace).  Same arguments and
 * requirements as rdb_linear_bwd_projected, bf16 layers, workspace of the RDB_OP_LINEAR_BWD_PROJECTED amount. */
int rdb_linear_bwd_projected_part(int part, void *dx, int64_t lddx, float *dcoef, const void *dy, int64_t lddy,
                                  const void *state, const void *coef, const rdb_linear_desc *desc, void *workspace,
                                  int64_t workspace_bytes, void *stream);

/* Tuning switch without a counterpart in the reference.  Layers with k > 256 whose products have enough 256 x 256 output
 * tiles to give every compute unit one run rdb_linear_fwd_projected / rdb_linear_project_fwd / rdb_linear_bwd_projected on
 * 256-wide tiles with one persistent block per compute unit; all others on 128-wide tiles.  mode 0: never the 256-wide
 * kernels; 1 (default): by that rule; 2: whenever k > 256 (for tests on small layers).  Both kinds contract in the same
 * order: y and dx are the same bit for bit; dcoef is contracted over all tokens in one pass by the 256-wide kernels, where the
 * 128-wide ones may add partial sums over token ranges (same values up to fp32 rounding).  Process-wide; returns the previous
 * mode. */
int rdb_set_big_tiles(int mode);

/* Tuning switch without a counterpart in the reference, for the products of fp32 layers (and of bf16 layers whose sizes are not
 * multiples of 8) and for the matrix-coef materialise products that run on the matrix cores.  mode 1 (default): every operand
 * value is split exactly into three bf16 parts (v = h + m + l, each the top 8 bits of what is left) on its way into LDS and a
 * product runs as six bf16 matrix instructions (ah bh + ah bm + am bh + ah bl + al bh + am bm, fp32 accumulation): the terms
 * left out are below 2^-23 of a product, an fp32 multiplication's own rounding, and the 32 x 32 x 16 bf16 instruction does in
 * 3/8 of the time what eight 32 x 32 x 2 fp32 ones do.  mode 0: fp32 matrix instructions.  Results agree to fp32 rounding;
 * with mode 1 an infinite input gives NaN where mode 0 gives an infinity.  Process-wide; returns the previous mode. */
int rdb_set_f32_split(int mode);

/* ------------------------------------------------------------------------------- one-launch forms and their bounded waits
 * No counterpart in the reference (its kernels are one launch per product).  rdb_linear_project_fwd / rdb_linear_fwd with
 * bf16 and k <= 256, and rdb_linear_fwd / rdb_linear_bwd_dx with fp32, k <= 64 and few tokens, run producer and consumer
 * blocks in ONE launch: consumers wait for per-tile tags that the producers publish.  The hardware is seen to hand out a
 * launch's blocks in index order, so a consumer never keeps the producers it waits for off the chip; this is observed, not
 * documented, so the wait is bounded (2^17 polls, a fraction of a second).  A block whose wait runs out does NOT compute: it
 * fills its share of the output (y or dx) with NaN, adds one to a per-device counter inside the library and leaves; for the
 * projected form it also sets bit 1 of the state's second 32-bit word.  The counter only ever grows.
 *
 * rdb_set_one_launch: mode 0 = never the one-launch forms (producers and consumers as separate launches: same results bit
 * for bit), 1 (default) = where they apply.  Process-wide; returns the previous mode.
 * rdb_sync_giveups_async: enqueues on `stream` a copy of the current device's counter to host_count (pinned host memory
 * if the copy is to be asynchronous); does not wait.  rdb_sync_giveups: the same, and waits for `stream`.
 * A caller that finds the counter changed must treat the outputs written since it last looked as invalid, and the
 * projection states and recorded graphs of those launches as unusable; switching to mode 0 avoids a repeat. */
int rdb_set_one_launch(int mode);
int rdb_sync_giveups_async(uint32_t *host_count, void *stream);
int rdb_sync_giveups(uint32_t *count, void *stream);

/* Test hook, no counterpart in the reference: runs ONLY the consumer blocks of a one-launch forward on `scratch` (bf16
 * layers: a projection state of rdb_linear_projection_bytes; fp32 layers: a forward workspace of rdb_linear_workspace_bytes)
 * with a tag that nobody publishes and a wait of `polls` polls, so that every block's wait runs out: y becomes NaN
 * throughout, the counter above grows by the number of blocks, every kernel ends normally. */
int rdb_selftest_sync_giveup(void *y, int64_t ldy, void *scratch, int64_t scratch_bytes, const void *coef,
                             const rdb_linear_desc *desc, int polls, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RANDUMB_HIP_H */
