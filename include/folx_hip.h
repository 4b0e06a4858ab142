/*
 * folx_hip.h -- C ABI of the MI355X (gfx950) forward-Laplacian kernel library.
 *
 * Every entry point propagates the triplet (x, jacobian, laplacian) of microsoft/folx
 * through one rule.  Conventions shared by all calls:
 *
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls are
 *     asynchronous on that stream, allocate nothing and never synchronise.
 *   - All data pointers are DEVICE pointers to contiguous float32 (index tables: int32).
 *   - Layout: value x[S], Jacobian jac[P][S] (Jacobian axis leading, reference JAC_DIM = 0,
 *     folx/api.py:16), Laplacian lap[S], where S flattens (walker, *shape) with the walker
 *     axis outermost.  For a sparse Jacobian P is the number of stored rows k; the int
 *     index mask lives on the host and never reaches the library except as gather tables.
 *   - Return value: FOLX_HIP_OK (0) or a negative FOLX_HIP_E* code; nothing is launched
 *     when an argument check fails.  folx_hip_strerror() names the code.
 *   - Unless stated, outputs must not alias inputs.
 */
#ifndef FOLX_HIP_H
#define FOLX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FOLX_HIP_OK 0
#define FOLX_HIP_EINVAL (-1)   /* null pointer, negative size, inconsistent shape      */
#define FOLX_HIP_ENOTSUP (-2)  /* size outside what the kernels are built for          */
#define FOLX_HIP_ELAUNCH (-3)  /* hipGetLastError() != hipSuccess after the launch     */
#define FOLX_HIP_ESCRATCH (-4) /* needs more than FOLX_HIP_STATIC_SCRATCH_BYTES of scratch */

/* Size of the library's own scratch array (folx_hip_norm_dense_static_fwdlap): 64 MiB of
 * device memory on every GPU the library has been used on, held until the process ends. */
#define FOLX_HIP_STATIC_SCRATCH_BYTES (64ll << 20)

/* Library version (major * 10000 + minor * 100 + patch). */
int folx_hip_version(void);
/* Static description of a return code. */
const char* folx_hip_strerror(int code);

/* How the wide dense rules (K % 16 == 0, N > 128, 16-byte aligned operands) form their fp32
 * products.  No counterpart in the reference, which leaves the choice to XLA
 * (jax.default_matmul_precision).
 *   FOLX_HIP_GEMM_F32    v_mfma_f32_32x32x2_f32 on the fp32 operands (the default).
 *   FOLX_HIP_GEMM_BF16X3 every operand element is split exactly into three bf16 pieces and a
 *                        product is the sum of the six piece products of weight >= 2^-16, each
 *                        exact, accumulated in fp32 on v_mfma_f32_32x32x16_bf16.  The dropped
 *                        terms weigh <= 2^-24 of a product, the rounding of one fp32
 *                        multiply-add, so results agree with the fp32 form to fp32 rounding;
 *                        inputs, outputs and accumulators stay fp32.  Kernels without a split
 *                        form run as under FOLX_HIP_GEMM_F32.  Where the two forms differ: an
 *                        infinite operand element (or one within 2^-9 of FLT_MAX, which rounds
 *                        to a bf16 infinity) gives NaN instead of an infinity, because its
 *                        remainder x - bf16(x) is inf - inf.
 * The mode is process wide and read at every launch; set it before launching, not while other
 * threads launch.  folx_hip_set_gemm_mode returns FOLX_HIP_EINVAL for any other value. */
#define FOLX_HIP_GEMM_F32 0
#define FOLX_HIP_GEMM_BF16X3 1
int folx_hip_set_gemm_mode(int mode);
int folx_hip_get_gemm_mode(void);

/* Elementwise functions of folx_hip_elementwise_fwdlap; the rule needs f, f', f''.
 * Replaces the per-primitive entries of folx/wrapped_functions.py:400-445, :552-556. */
enum folx_hip_act {
  FOLX_ACT_TANH = 0,
  FOLX_ACT_SILU = 1,
  FOLX_ACT_EXP = 2,
  FOLX_ACT_LOG = 3,
  FOLX_ACT_SQRT = 4,
  FOLX_ACT_RSQRT = 5,
  FOLX_ACT_SQUARE = 6,
  FOLX_ACT_LOGISTIC = 7,
  FOLX_ACT_SOFTPLUS = 8,
  FOLX_ACT_SIN = 9,
  FOLX_ACT_COS = 10,
  FOLX_ACT_ABS = 11,
  FOLX_ACT_LOG1P = 12,
  FOLX_ACT_RECIPROCAL = 13,
  FOLX_ACT_EXPM1 = 14,
  FOLX_ACT_INTEGER_POW = 15, /* param = exponent (integer value) */
  FOLX_ACT_SINH = 16,
  FOLX_ACT_COSH = 17,
  FOLX_ACT_TAN = 18,
  FOLX_ACT_ASIN = 19,
  FOLX_ACT_ACOS = 20,
  FOLX_ACT_ATAN = 21,
  FOLX_ACT_ASINH = 22,
  FOLX_ACT_ACOSH = 23,
  FOLX_ACT_ATANH = 24,
  FOLX_ACT_ERF = 25,
  FOLX_ACT_ERFC = 26,
  FOLX_ACT_ERF_INV = 27,
  FOLX_ACT_CBRT = 28,
  FOLX_ACT_POW = 29, /* x^param for x > 0, param = constant real exponent (jax.lax.pow_p) */
  FOLX_ACT_LGAMMA = 30,  /* log|Gamma(x)|, derivatives digamma and trigamma (jax.lax.lgamma_p) */
  FOLX_ACT_DIGAMMA = 31, /* derivatives trigamma and tetragamma (jax.lax.digamma_p) */
  FOLX_ACT_COUNT = 32
};

/* Binary functions of folx_hip_binary_fwdlap. */
enum folx_hip_binop {
  FOLX_BIN_MUL = 0, /* jax.lax.mul, MULTIPLICATION rule (folx/hessian.py:177-188)   */
  FOLX_BIN_DIV = 1, /* jax.lax.div, custom Hessian (folx/custom_hessian.py:35-59)   */
  FOLX_BIN_ADD = 2, /* jax.lax.add, LINEAR                                          */
  FOLX_BIN_SUB = 3, /* jax.lax.sub, LINEAR                                          */
  FOLX_BIN_MIN = 4, /* jax.lax.min: the smaller operand's triplet, half of each at a tie */
  FOLX_BIN_MAX = 5, /* jax.lax.max (both LINEAR, folx/wrapped_functions.py:508-513)      */
  FOLX_BIN_COUNT = 6
};

/*
 * Dense layer y = h @ W (+ bias) applied to the stacked operand [x; J; lap].
 * Replaces _dot_general_one_constant, folx/wrapped_functions.py:71-171 (the three
 * dot_generals at :167-169) for a constant right operand contracted with the last axis.
 *   x   [R][K]      jac [P][R][K]     lap [R][K]       R = walkers * positions
 *   W   [K][N] row-major, shared by all rows;  bias [N] or NULL (added to y only)
 *   res [R][N]      res_jac [P][R][N] res_lap [R][N]   optional residual triplet (all three
 *       NULL or all three set) added in the epilogue: the `add` rule that follows a
 *       residual branch (LINEAR, folx/wrapped_functions.py:365-367) fused into the GEMM
 *   y   [R][N]      y_jac [P][R][N]   y_lap [R][N]
 * One launch covers all (P + 2) * R rows (FP32 MFMA, fp32 accumulate).
 */
int folx_hip_dense_fwdlap(void* stream, const float* x, const float* jac, const float* lap,
                          const float* W, const float* bias, const float* res,
                          const float* res_jac, const float* res_lap, float* y, float* y_jac,
                          float* y_lap, int64_t R, int32_t P, int32_t K, int32_t N);

/*
 * The same dense layer reading its input rows in groups: logical row r of x (and of every
 * Jacobian row, and of lap) sits at physical row (r / group) * group_stride + r % group,
 * counted from the pointer passed in.  That is a slice along the axis in front of the
 * feature axis (e.g. the spin-up electrons of [B][n][K]: group = n_up, group_stride = n)
 * consumed in place.  R counts logical rows and is a multiple of group; in jac the row
 * groups of consecutive Jacobian rows follow each other at the same stride.  group = 0 means
 * contiguous rows (folx_hip_dense_fwdlap).  Outputs and the residual are contiguous.
 * Replaces a jax.lax.slice feeding _dot_general_one_constant (folx/wrapped_functions.py:71-171).
 */
int folx_hip_dense_rows_fwdlap(void* stream, const float* x, const float* jac, const float* lap,
                               const float* W, const float* bias, const float* res,
                               const float* res_jac, const float* res_lap, float* y, float* y_jac,
                               float* y_lap, int64_t R, int32_t P, int32_t K, int32_t N,
                               int64_t group, int64_t group_stride);

/*
 * Elementwise activation rule  y = f(x), y_jac[p] = f'(x) * jac[p],
 * y_lap = f'(x) * lap + f''(x) * sum_p jac[p]^2   in one pass over the Jacobian.
 * Replaces dense_elementwise_jvp (folx/jvp.py:687-697), the single-argument branch of
 * sparse_diag_jvp (folx/jvp.py:262-272) and elementwise_jhj_trace (folx/hessian.py:87-112),
 * combined as in folx/wrapper.py:120-125.  In-place use (y == x, y_jac == jac,
 * y_lap == lap) is allowed.
 */
int folx_hip_elementwise_fwdlap(void* stream, int32_t act, float param, const float* x,
                                const float* jac, const float* lap, float* y, float* y_jac,
                                float* y_lap, int64_t S, int32_t P);

/*
 * Exponential envelope  y[r][o] = sum_I pi[I][o] exp(-sigma[I][o] d[r][I])  of a triplet d with
 * n_cols <= 8 columns and constant sigma, pi [n_cols][O]: the chain broadcast_in_dim, mul,
 * neg, exp, mul, reduce_sum that the reference interprets rule by rule (elementwise rules
 * folx/jvp.py:687-697 / folx/hessian.py:87-112 around LINEAR ones, folx/wrapped_functions.py:361-392)
 * and XLA fuses afterwards, as one pass that only writes the result.
 *   d [R][n_cols]  d_jac [P][R][n_cols]  d_lap [R][n_cols]   y [R][O]  y_jac [P][R][O]  y_lap [R][O]
 * O % 4 == 0.  For a sparse d_jac the rows must not name an index twice per position (the rule
 * uses sum_p d_jac[p]^2 as in folx/hessian.py:460-470).
 */
int folx_hip_exp_envelope_fwdlap(void* stream, const float* d, const float* d_jac,
                                 const float* d_lap, const float* sigma, const float* pi, float* y,
                                 float* y_jac, float* y_lap, int64_t R, int32_t n_cols, int32_t O,
                                 int32_t P);

/*
 * Dense layer followed by its activation as one rule:
 *   y = f(x @ W + bias),  y_jac[p] = f'(z) * (jac[p] @ W),
 *   y_lap = f'(z) * (lap @ W) + f''(z) * sum_p (jac[p] @ W)^2,      z = x @ W + bias.
 * The composition of _dot_general_one_constant (folx/wrapped_functions.py:71-171) with the
 * elementwise rule (folx/jvp.py:687-697, folx/hessian.py:87-112, folx/wrapper.py:120-125)
 * that follows it in every Dense + activation layer; the pre-activation Jacobian is never
 * written.  Layouts as in folx_hip_dense_fwdlap.  Built for narrow layers (4 <= K <= 128 with
 * K % 4 == 0, N <= 128) and for wide ones (N > 128 with N % 4 == 0, K % 16 == 0, R % 4 == 0,
 * P >= 1), 16-byte aligned operands and act in {TANH, SILU, LOGISTIC, SOFTPLUS, EXP, SIN,
 * COS, SQUARE}; anything else returns FOLX_HIP_ENOTSUP and the caller uses the two separate
 * rules.  Outputs must not overlap inputs.
 * res / res_jac / res_lap (all or none; shapes of y / y_jac / y_lap) are added to the activated
 * result -- the skip connection of a residual layer (add_p, LINEAR, folx/wrapped_functions.py:365-367);
 * narrow layers only (FOLX_HIP_ENOTSUP for a wide one: folx_hip_dense_act_parts_fwdlap takes it).
 * workspace: folx_hip_dense_act_workspace_bytes(R, P, K, N) bytes of device memory (0 for a
 * narrow layer with large R: then it may be NULL), contents irrelevant; it holds partial sums
 * over Jacobian rows between launches.  The query returns a negative code for unsupported
 * shapes.
 */
int64_t folx_hip_dense_act_workspace_bytes(int64_t R, int32_t P, int32_t K, int32_t N);
int folx_hip_dense_act_fwdlap(void* stream, int32_t act, float param, const float* x,
                              const float* jac, const float* lap, const float* W,
                              const float* bias, const float* res, const float* res_jac,
                              const float* res_lap, float* y, float* y_jac, float* y_lap,
                              int64_t R, int32_t P, int32_t K, int32_t N, void* workspace,
                              int64_t workspace_bytes);

/*
 * folx_hip_dense_act_fwdlap for a wide layer whose input is a concatenation along the feature
 * axis that is never formed: part i contributes widths[i] consecutive features (multiples of
 * 16, at most 8 parts, K = their sum), jac_parts[i] is its Jacobian [P][rows_i][widths[i]]
 * with rows_i = R, or R / group when broadcast[i] is set: then the part has one row per
 * `group` consecutive rows of the layer (a per-walker feature shown to every electron,
 * jax.lax.broadcast_in_dim before jax.lax.concatenate in the reference's trace; rules
 * folx/wrapped_functions.py:361-376 on the way into _dot_general_one_constant, :71-171).
 * x and lap are the concatenated [R][K] arrays (1 / (P + 2) of the data; only the Jacobian
 * is read in parts).  jac_parts, widths and broadcast are HOST arrays.  Same shapes,
 * activations and workspace as the wide path of folx_hip_dense_act_fwdlap
 * (folx_hip_dense_act_workspace_bytes(R, P, K, N)); FOLX_HIP_ENOTSUP otherwise.
 * res / res_jac / res_lap (all or none; shapes of y / y_jac / y_lap) are added to the
 * activated result: the skip connection of a residual layer (add_p after the activation).
 * pre [R / group][N], pre_jac [P][R / group][N], pre_lap [R / group][N] (all or none) are added
 * to the PRE-activation triplet, row r taking row r / group: the product of the per-walker
 * (broadcast) features with their rows of the weight matrix, computed once per walker by the
 * caller (folx_hip_dense_fwdlap on R / group rows) instead of once per position -- the parts
 * passed here are then only the per-position ones, with their rows of W.
 */
int folx_hip_dense_act_parts_fwdlap(void* stream, int32_t act, float param, const float* x,
                                    const float* lap, int32_t n_parts,
                                    const float* const* jac_parts, const int32_t* widths,
                                    const int32_t* broadcast, int32_t group, const float* W,
                                    const float* bias, const float* res, const float* res_jac,
                                    const float* res_lap, const float* pre, const float* pre_jac,
                                    const float* pre_lap, float* y, float* y_jac, float* y_lap,
                                    int64_t R, int32_t P, int32_t N, void* workspace,
                                    int64_t workspace_bytes);

/*
 * LayerNorm over the K features, then a dense layer, then (act >= 0) an activation, as one
 * rule:  y = f(LN(x) @ W + bias),  LN(x) = gamma * (x - mean) * rsqrt(var + eps) + beta.
 * The triplet that results is the one of folx_hip_layernorm_fwdlap followed by
 * folx_hip_dense_fwdlap and folx_hip_elementwise_fwdlap (the reference interprets the same
 * chain of primitives, folx/wrapped_functions.py:71-171, :361-415); neither LN's Jacobian
 * nor the pre-activation Jacobian is written.  The Jacobian rows are multiplied RAW with
 * diag(gamma) W and LayerNorm's projection is applied to the product as a rank-2 correction
 * per row, so rows whose mean dwarfs their variation lose digits they would keep in the
 * three-step form.
 *   x [R][K]  jac [P][R][K]  lap [R][K]  gamma, beta [K] or NULL  W [K][N]  bias [N] or NULL
 *   ->  y [R][N]  y_jac [P][R][N]  y_lap [R][N];  act = -1: no activation.
 * Built for N > 128 with N % 4 == 0, K % 16 == 0, K <= 512, R % 4 == 0, P >= 1, 16-byte aligned
 * operands and the activations of folx_hip_dense_act_fwdlap; anything else returns
 * FOLX_HIP_ENOTSUP.  workspace: folx_hip_norm_dense_workspace_bytes(R, P, K, N, act) bytes,
 * contents irrelevant.  Outputs must not overlap inputs.
 */
int64_t folx_hip_norm_dense_workspace_bytes(int64_t R, int32_t P, int32_t K, int32_t N, int32_t act);
int folx_hip_norm_dense_fwdlap(void* stream, int32_t act, float param, const float* x,
                               const float* jac, const float* lap, const float* gamma,
                               const float* beta, float eps, const float* W, const float* bias,
                               float* y, float* y_jac, float* y_lap, int64_t R, int32_t P,
                               int32_t K, int32_t N, void* workspace, int64_t workspace_bytes);

/*
 * folx_hip_norm_dense_fwdlap without a workspace argument, for callers that cannot allocate
 * device memory: code under HIP graph capture, serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference (jax owns all memory there).  Same arguments, shape
 * limits, kernels and bit-for-bit the same results as folx_hip_norm_dense_fwdlap; the
 * partial sums and per-position rows live in a device array of FOLX_HIP_STATIC_SCRATCH_BYTES
 * that is part of the library's code object (one copy per GPU).  The call allocates and frees
 * nothing.  Shapes whose folx_hip_norm_dense_workspace_bytes() exceeds that size return
 * FOLX_HIP_ESCRATCH and launch nothing (R = 4096 rows at P = 96, K = N = 256 with an
 * activation need 36 MiB; the size grows linearly in R).  All calls on one GPU share the
 * array: calls that may overlap in time on one GPU (different streams, or threads) race and
 * must be serialised by the caller; calls on one stream are ordered and safe.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress), so make that call outside a
 * graph capture.
 */
int folx_hip_norm_dense_static_fwdlap(void* stream, int32_t act, float param, const float* x,
                                      const float* jac, const float* lap, const float* gamma,
                                      const float* beta, float eps, const float* W,
                                      const float* bias, float* y, float* y_jac, float* y_lap,
                                      int64_t R, int32_t P, int32_t K, int32_t N);

/*
 * Matrix product of two operands that both carry derivatives, for a batch of NB0 * NB1 matrix
 * pairs a (I x Kc), b (Kc x J) with dense Jacobians on the same P rows:
 *   y = a b,   y_jac[p] = a_jac[p] b + a b_jac[p],
 *   y_lap = a_lap b + a b_lap + 2 sum_p a_jac[p] b_jac[p].
 * Replaces the two-operand paths of dot_general (folx/wrapped_functions.py:205-309: rearrange
 * :47-68 + the dot_last einsum :294-309 under dense_split_jvp, folx/jvp.py:676-684) with the
 * DOT_PRODUCT Hessian term 2 tr(J_l J_r^T) (dot_product_jac_hessian_jac, folx/hessian.py:177-188);
 * the (batch, i, j, k) broadcast intermediate of that path is never formed.
 * Operands are addressed through element strides (HOST array of 10 non-negative values):
 *   strides = {a_sb0, a_sb1, a_si, a_sk, a_sp,  b_sb0, b_sb1, b_sk, b_sj, b_sp}
 *   a(b0, b1, i, k) at a[b0 a_sb0 + b1 a_sb1 + i a_si + k a_sk], likewise a_lap; Jacobian row p
 *   adds p * a_sp.  b(b0, b1, k, j) at b[b0 b_sb0 + b1 b_sb1 + k b_sk + j b_sj], rows p * b_sp.
 * so that transposed operands (q k^T) and head-interleaved layouts ([walker][electron][head][d]
 * read as batch (walker, head)) need no copy.  Outputs are contiguous:
 *   y, y_lap [NB0][NB1][I][J]   y_jac [P][NB0][NB1][I][J].
 * Built for Kc <= 128 (FOLX_HIP_ENOTSUP beyond; the caller then multiplies and sums).
 * b_jac == NULL and b_lap == NULL: b is a constant with batch axes (per-head weight matrices,
 * a stride of 0 on the axes it does not vary along), the case of _dot_general_one_constant in
 * which the constant operand has batch dimensions (folx/wrapped_functions.py:71-171, the three
 * products at :167-169): y = a b, y_jac[p] = a_jac[p] b, y_lap = a_lap b.
 */
int folx_hip_dot_two_fwdlap(void* stream, const float* a, const float* a_jac, const float* a_lap,
                            const float* b, const float* b_jac, const float* b_lap, float* y,
                            float* y_jac, float* y_lap, int64_t NB0, int32_t NB1, int32_t I,
                            int32_t J, int32_t Kc, int32_t P, const int64_t* strides);

/*
 * Binary elementwise rule for two operands whose Jacobians live on the same row frame
 * (both dense with P rows, or sparse with identical index masks).  The output index
 * space is (n0, n1, n2), row-major; each operand addresses it with element strides
 * sa / sb (0 = broadcast).  dims = {n0, n1, n2, sa0, sa1, sa2, sb0, sb1, sb2} is a HOST
 * array.  a_S / b_S are the element counts of one Jacobian row of a / b.
 * MUL: y = a b, y_jac = a b_jac + b a_jac, y_lap = a b_lap + b a_lap + 2 sum_p a_jac b_jac
 * Replaces dense_split_jvp (folx/jvp.py:676-684) + dot_product_jac_hessian_jac
 * (folx/hessian.py:177-188) / div_jac_hessian_jac (folx/custom_hessian.py:35-59).
 */
int folx_hip_binary_fwdlap(void* stream, int32_t op, const float* a, const float* a_jac,
                           const float* a_lap, const float* b, const float* b_jac,
                           const float* b_lap, float* y, float* y_jac, float* y_lap,
                           const int64_t* dims, int64_t a_S, int64_t b_S, int32_t P);

/*
 * Product of two triplets of one shape, a with a dense Jacobian (P rows) and b with a sparse
 * one (k_rows rows): slot s of element i stands for the dense row index[s][i % S_w]
 * (int32 [k_rows][S_w], S_w = elements per walker, -1 = empty slot, no row named twice per
 * element, all < P).  The case of FwdJacobian.__add__ with one dense operand
 * (folx/api.py:233-236) inside the mul rule (folx/wrapped_functions.py:375-377,
 * folx/hessian.py:177-188), without first densifying b.
 *   a, b, *_lap, y, y_lap [S]   a_jac, y_jac [P][S]   b_jac [k_rows][S]      k_rows <= 8
 */
int folx_hip_mul_sparse_fwdlap(void* stream, const float* a, const float* a_jac,
                               const float* a_lap, const float* b, const float* b_jac,
                               const float* b_lap, const int32_t* index, float* y, float* y_jac,
                               float* y_lap, int64_t S, int64_t S_w, int32_t P, int32_t k_rows);

/*
 * Fused LayerNorm over the last axis, y = gamma * (x - mean) * rsqrt(var + eps) + beta,
 * for R rows of F features (F % 4 == 0, F <= 1024); gamma / beta [F] or NULL.
 *   x [R][F]   jac [P][R][F]   lap [R][F]   ->   y, y_jac, y_lap of the same shapes.
 * The reference has no LayerNorm rule of its own: it interprets the primitive chain
 * reduce_sum / sub / square / reduce_sum / rsqrt / mul / add with the LINEAR, elementwise
 * and MULTIPLICATION rules (folx/wrapped_functions.py:361-415, folx/hessian.py:87-112,
 * :177-188); this entry point evaluates that chain's closed form in one pass.  For a
 * sparse Jacobian the mask must be constant along the feature axis (rows then keep it).
 */
int folx_hip_layernorm_fwdlap(void* stream, const float* x, const float* jac, const float* lap,
                              const float* gamma, const float* beta, float* y, float* y_jac,
                              float* y_lap, int64_t R, int32_t F, int32_t P, float eps);

/*
 * Row-stack affine map with broadcast coefficient arrays:
 *   out[r][i] = alpha * in[r][ia(i)] * (c ? c[ic(i)] : 1) + (d ? beta * d[id(i)] : 0)
 * over rows r < rows and the index space (n0, n1, n2).  dims = {n0, n1, n2, sin0..2,
 * sc0..2, sd0..2} is a HOST array of element strides; in_S is the element count of one
 * input row.  Used for every LINEAR rule against constants (add, sub, neg, scaling by a
 * constant, folx/wrapped_functions.py:361-376) on x, on the Jacobian rows and on lap.
 */
int folx_hip_rows_affine(void* stream, const float* in, float* out, int64_t rows,
                         int64_t in_S, const float* c, const float* d, float alpha,
                         float beta, const int64_t* dims);

/*
 * Sum over the middle axis: in [rows][outer][red][inner] -> out [rows][outer][inner],
 * scaled by alpha.  The reduce_sum rule is linear and is applied to x, jac and lap alike
 * (SUMMATION, folx/wrapped_functions.py:388-392; folx/jvp.py:104-106).
 */
int folx_hip_reduce_sum(void* stream, const float* in, float* out, int64_t rows,
                        int64_t outer, int64_t red, int64_t inner, float alpha);

/*
 * The same sum over a window [lo, hi) of the middle axis, read where it lies:
 * in [rows][outer][span][inner] -> out [rows][outer][inner] = alpha * sum_{lo <= r < hi}.
 * A slice (slice_p, folx/wrapped_functions.py:446-466) whose only consumer is reduce_sum_p:
 * spin-wise means over the electron axis.
 */
int folx_hip_reduce_sum_window(void* stream, const float* in, float* out, int64_t rows,
                               int64_t outer, int64_t span, int64_t lo, int64_t hi,
                               int64_t inner, float alpha);

/* max over the middle axis of a value array (no derivatives): [outer][red][inner] ->
 * [outer][inner].  Used for the stop-gradient shift of logsumexp. */
int folx_hip_reduce_max(void* stream, const float* in, float* out, int64_t outer,
                        int64_t red, int64_t inner);

/*
 * Re-index sparse Jacobian rows into another row frame by a static gather table:
 *   out[t][b][so][si] = sum_{s < n_slots} ( r = take[(t * n_slots + s) * S_outer + so];
 *                                           r >= 0 ? data[r][b][so][si] : 0 )
 * data [k_in][B][S_outer][S_inner], take int32 [k_out][n_slots][S_outer] with values in
 * [-1, k_in).  Replaces materialize_by_gather (folx/utils.py:71-114) as used by
 * FwdJacobian.materialize_for_idx (folx/api.py:58-118), get_jacobian_for_reduction
 * (folx/utils.py:499-588) and sparse_sum_jvp (folx/jvp.py:163-171).
 */
int folx_hip_gather_rows(void* stream, const float* data, const int32_t* take, float* out,
                         int32_t k_in, int32_t k_out, int32_t n_slots, int64_t B,
                         int64_t S_outer, int64_t S_inner);

/*
 * The same re-indexing with a sum over one axis of the data folded in (sparse_sum_jvp,
 * folx/jvp.py:89-176, for slots that vary along the reduced axis; what _factorized_dense_row_sum,
 * folx/jvp.py:37-86, reaches with a gather after regrouping).  The data keeps its own layout
 * [k_in][B][O][RED][IV][IC] -- the reduced axis in the middle -- and a source is a (row r, entry j
 * of the reduced axis) pair encoded r * RED + j:
 *   out[t][b][o][iv][ic] = alpha * sum_{s < n_slots} ( e = take[(t * n_slots + s) * O * IV + o * IV + iv];
 *                                                      e >= 0 ? data[e / RED][b][o][e % RED][iv][ic] : 0 )
 * take int32 [k_out][n_slots][O][IV] with values in [-1, k_in * RED); out [k_out][B][O][IV][IC].
 * A window of the reduced axis (a slice_p in front of the sum) is a table that names no entry
 * outside it; alpha is the 1 / n of a mean.
 */
int folx_hip_gather_reduce_rows(void* stream, const float* data, const int32_t* take, float* out,
                                int32_t k_in, int32_t k_out, int32_t n_slots, int64_t B, int64_t O,
                                int32_t RED, int64_t IV, int64_t IC, float alpha);

/*
 * Static gather along the position axis with a sum over slots -- the transposed form of a
 * scatter with static indices, in which every output position lists the input positions
 * that land on it:
 *   out[rb][po][si] = sum_{s < n_slots} ( t = table[po * n_slots + s];
 *                                         t >= 0 ? data[rb][t][si] : 0 )
 * data [RB][S_in_outer][S_inner], table int32 [S_out_outer][n_slots] with values in
 * [-1, S_in_outer), out [RB][S_out_outer][S_inner]; RB = (triplet rows) x (walkers).
 * The arithmetic of the scatter rules (scatter / scatter-add / scatter_min / scatter_max,
 * sparse_scatter_jvp, folx/jvp.py:474-673) and of integer-array indexing.
 */
int folx_hip_gather_cols(void* stream, const float* data, const int32_t* table, float* out,
                         int64_t RB, int64_t S_in_outer, int64_t S_out_outer, int32_t n_slots,
                         int64_t S_inner);

/*
 * Scatter-add form of the same re-indexing (the reference's segment_sum fallback,
 * folx/api.py:110-114, folx/jvp.py:170-171), accumulating into what out already holds (zeros
 * for a plain re-indexing, a dense row stack for a sparse Jacobian added to it in place,
 * folx/api.py:230-236):
 *   out[idx[r][so]][b][so][si] += data[r][b][so][si]   for 0 <= idx < k_out.
 * idx int32 [k_in][S_outer].  Every output entry is updated by one thread in row order: no
 * atomics, identical bits on every run, also when rows of a position share a target.
 */
int folx_hip_scatter_add_rows(void* stream, const float* data, const int32_t* idx,
                              float* out, int32_t k_in, int32_t k_out, int64_t B,
                              int64_t S_outer, int64_t S_inner);

/*
 * slogdet rule for NM matrices of size n x n (n <= 32) with dense Jacobians.
 *   A [NM][n][n]   A_jac [P][NM][n][n]   A_lap [NM][n][n]
 *   sign [NM]   logdet [NM]   ld_jac [P][NM]   ld_lap [NM]
 * sign/logdet by LU with partial pivoting; M_p = A^-1 A_jac[p]; ld_jac[p] = tr M_p;
 * ld_lap = tr(A^-1 A_lap) - sum_p tr(M_p M_p).
 * Replaces _dense_log_det / dense_slogdet (folx/slogdet.py:296-344).
 */
int folx_hip_slogdet_fwdlap(void* stream, const float* A, const float* A_jac,
                            const float* A_lap, float* sign, float* logdet, float* ld_jac,
                            float* ld_lap, int64_t NM, int32_t n, int32_t P);

/*
 * The same slogdet rule on matrices read in place from a strided stack: matrix
 * (b, d), b < NB, d < ND, has element (i, j) at
 *     b * batch_stride + d * member_stride + i * row_stride + j          (in floats)
 * of A and A_lap, and at p * jac_stride + the same offset of A_jac.  Outputs are ordered
 * [b][d] ([P][NB][ND] for ld_jac).  The orbital matrices of a dense layer's output
 * [B][electron][determinant][orbital] are such a stack (member_stride = n,
 * row_stride = ND * n, batch_stride = n * ND * n): no transposed copy is needed in front
 * of folx/slogdet.py:296-344.
 */
int folx_hip_slogdet_strided_fwdlap(void* stream, const float* A, const float* A_jac,
                                    const float* A_lap, float* sign, float* logdet, float* ld_jac,
                                    float* ld_lap, int64_t NB, int64_t ND, int32_t n, int32_t P,
                                    int64_t batch_stride, int64_t member_stride, int64_t row_stride,
                                    int64_t jac_stride);

/*
 * slogdet of the elementwise product A * F, where F is a triplet of A's layout whose Jacobian
 * is sparse: F_jac [k_rows][..] with row stride jac_stride, slot s of the element at
 * per-walker position q standing for dense row index[s][q] (int32 [k_rows][walker_elems], -1 =
 * empty, all < P, no row named twice per element).  The mul rule (folx/wrapped_functions.py:375-377)
 * applied on the fly in front of slogdet_wrapper (folx/slogdet.py:347-358): orbitals times
 * envelopes never exist as a tensor.  Other arguments as in folx_hip_slogdet_strided_fwdlap.
 * Built for n <= 16 and k_rows <= 4; FOLX_HIP_ENOTSUP otherwise.
 */
int folx_hip_slogdet_scaled_fwdlap(void* stream, const float* A, const float* A_jac,
                                   const float* A_lap, const float* F, const float* F_jac,
                                   const float* F_lap, const int32_t* index, float* sign,
                                   float* logdet, float* ld_jac, float* ld_lap, int64_t NB,
                                   int64_t ND, int32_t n, int32_t P, int64_t batch_stride,
                                   int64_t member_stride, int64_t row_stride, int64_t jac_stride,
                                   int64_t walker_elems, int32_t k_rows);

/*
 * slogdet rule for a sparse Jacobian whose coordinates touch few rows, columns or entries
 * of A, from static rank-one factor tables shared by all NM matrices.
 *   A [NM][n][n]   A_jac [k][NM][n][n] (k stored rows)   A_lap [NM][n][n]
 *   take  int32 [n_coords][rank][width]: address t * n * n + r * n + c of a factor entry in
 *         (stored row t, matrix row r, column c) of A_jac, or -1 for an unused slot
 *   cols  int32 [n_coords][rank][width]: the column the entry contracts with
 *   rows  int32 [n_coords][rank]: the matrix row of every factor
 *   sign [NM]   logdet [NM]   ld_jac [n_coords][NM] (row c belongs to the c-th coordinate of
 *   the tables)   ld_lap [NM]
 * W_c[s][t] = sum_l A_jac[take[c][s][l]] * Ainv[cols[c][s][l]][rows[c][t]];
 * ld_jac[c] = tr W_c;  ld_lap = tr(Ainv A_lap) - sum_c sum_st W_c[s][t] W_c[t][s].
 * transposed != 0: the tables were built for A^T (cols are rows of A and vice versa; take
 * still addresses A_jac as stored) and Ainv is read transposed.
 * Limits: n <= 32, rank <= 64, rank * width <= 2048 (else FOLX_HIP_ENOTSUP).
 * Replaces _sparse_slogdet / _pack_slogdet (folx/slogdet.py:182-246); the tables are the
 * ones of _factor_tables (folx/slogdet.py:142-179).
 */
int folx_hip_sparse_slogdet_fwdlap(void* stream, const float* A, const float* A_jac,
                                   const float* A_lap, const int32_t* take, const int32_t* cols,
                                   const int32_t* rows, float* sign, float* logdet, float* ld_jac,
                                   float* ld_lap, int64_t NM, int32_t n, int32_t k,
                                   int32_t n_coords, int32_t rank, int32_t width, int32_t transposed);

/*
 * Building blocks of the slogdet / det / inverse / solve rules for matrices of ANY size n (the
 * rule kernels below and above stop at 32 x 32; the reference reaches LAPACK through
 * jnp.linalg.slogdet / inv for every size, folx/slogdet.py:311-312, folx/linear_solve.py:124).
 * A, Ainv [NM][n][n] (different buffers), sign, logdet [NM]:
 *   Ainv = A^-1 by Gauss-Jordan elimination with partial pivoting (the pivot sequence of an LU
 *   factorisation with partial pivoting: same sign), sign = sign(det A), logdet = log|det A|.
 * The caller composes the rules from it and the batched product kernels:
 *   M_c = Ainv A_jac[c],  ld_jac[c] = tr M_c,  ld_lap = tr(Ainv A_lap) - sum_c tr(M_c M_c)
 *   (folx/slogdet.py:313-316);  C_jac[c] = -M_c Ainv,  C_lap = (2 sum_c M_c M_c - Ainv A_lap) Ainv
 *   (folx/linear_solve.py:125-140).
 */
int folx_hip_inv_values(void* stream, const float* A, float* Ainv, float* sign, float* logdet,
                        int64_t NM, int32_t n);

/*
 * tr[r] = tr M_r and trsq[r] = tr(M_r M_r) = sum_ij M_r[i][j] M_r[j][i] for a stack M [R][n][n]: the
 * two contractions the slogdet rule takes of M_c = A^-1 d_c A, any n
 * (jnp.einsum('k...ii->k...') and ('k...id,k...di->...'), folx/slogdet.py:314-316).
 */
int folx_hip_trace_pair(void* stream, const float* M, float* tr, float* trsq, int64_t R, int32_t n);

/*
 * Inverse rule for NM matrices of size n x n (n <= 32) with dense Jacobians.
 *   A, A_lap, C, C_lap [NM][n][n]   A_jac, C_jac [P][NM][n][n]
 * C = A^-1;  M_p = C A_jac[p];  C_jac[p] = -M_p C;  C_lap = (2 sum_p M_p M_p - C A_lap) C.
 * Replaces inv_wrapper (folx/linear_solve.py:114-145).
 */
int folx_hip_inv_fwdlap(void* stream, const float* A, const float* A_jac, const float* A_lap,
                        float* C, float* C_jac, float* C_lap, int64_t NM, int32_t n, int32_t P);

/*
 * Linear-solve rule y = A^-1 b for NM systems, n <= 32 unknowns, m <= 32 right-hand sides.
 *   A [NM][n][n]   b, y [NM][n][m]   *_jac [P][NM][...]   *_lap like the values
 * A_jac/A_lap or b_jac/b_lap may both be NULL for a constant operand (not both operands);
 * a NULL Laplacian is what marks an operand as constant (with P = 0 no Jacobian is read).
 *   A y_jac[p] = b_jac[p] - A_jac[p] y
 *   A y_lap    = b_lap - A_lap y - 2 sum_p A_jac[p] y_jac[p]
 * Replaces solve_wrapper (folx/linear_solve.py:54-111).
 */
int folx_hip_solve_fwdlap(void* stream, const float* A, const float* A_jac, const float* A_lap,
                          const float* b, const float* b_jac, const float* b_lap, float* y,
                          float* y_jac, float* y_lap, int64_t NM, int32_t n, int32_t m, int32_t P);

/*
 * Multi-head self attention with Laplacian, o = softmax(q k^T) v (no 1/sqrt(d) inside).
 *   q, k, v, their lap and o, o_lap: [B][n][H][d];  *_jac, o_jac: [P][B][n][H][d]
 *   mask uint8 [B][n] (1 = real electron) or NULL; input_mask uint8 [P][B]
 *   (1 = active coordinate) or NULL.
 * Replaces mhsa_forward_laplacian and its Pallas kernel
 * (folx/experimental/pallas/attention/forward_laplacian.py:27-179, :349-487).
 * Supported: n <= 64, d <= 64, d % 4 == 0.
 */
int folx_hip_mhsa_fwdlap(void* stream, const float* q, const float* q_jac, const float* q_lap,
                         const float* k, const float* k_jac, const float* k_lap,
                         const float* v, const float* v_jac, const float* v_lap,
                         const uint8_t* mask, const uint8_t* input_mask, float* o,
                         float* o_jac, float* o_lap, int64_t B, int32_t n, int32_t H,
                         int32_t d, int32_t P);

/*
 * The same attention rule (no masks, no edge bias) for q, k, v whose Jacobians are still
 * sparse by position: sequence position e depends on at most k_rows input coordinates of its
 * own, index[s][e] (int32 [k_rows][n], shared by all walkers and heads, -1 = empty slot)
 * naming the dense Jacobian row that slot s of position e stands for; no dense row may be
 * named twice.  What folx reaches by materialising the three Jacobians first
 * (folx/experimental/pallas/attention/forward_laplacian.py:166-178 on top of
 * FwdJacobian.dense_array, folx/api.py:182-190) -- here the zero rows are never built and the
 * per-row n x n x d products collapse to vector work.
 *   q, k, v [B][n][H][d]   *_jac [k_rows][B][n][H][d]   *_lap [B][n][H][d]
 *   o [B][n][H][d]   o_jac [P][B][n][H][d] (dense; only the rows named in index are written,
 *   the caller zero-fills the others)   o_lap [B][n][H][d]
 * Built for n <= 64, d <= 64 with d % 4 == 0, k_rows <= 8; FOLX_HIP_ENOTSUP otherwise.
 */
int folx_hip_mhsa_sparse_fwdlap(void* stream, const float* q, const float* q_jac,
                                const float* q_lap, const float* k, const float* k_jac,
                                const float* k_lap, const float* v, const float* v_jac,
                                const float* v_lap, const int32_t* index, float* o, float* o_jac,
                                float* o_lap, int64_t B, int32_t n, int32_t H, int32_t d,
                                int32_t k_rows);

/*
 * Edge-bias variant: o = softmax(q k^T + e) v with e, e_lap [B][n][H][n], e_jac [P][B][n][H][n]
 * (argument order q, k, e, v as in the reference's rule).  Replaces mhsea_forward_laplacian
 * and its Pallas kernel (folx/experimental/pallas/attention/forward_laplacian.py:495-614,
 * :745-854).  Same size limits as folx_hip_mhsa_fwdlap.
 */
int folx_hip_mhsea_fwdlap(void* stream, const float* q, const float* q_jac, const float* q_lap,
                          const float* k, const float* k_jac, const float* k_lap,
                          const float* e, const float* e_jac, const float* e_lap,
                          const float* v, const float* v_jac, const float* v_lap,
                          const uint8_t* mask, const uint8_t* input_mask, float* o,
                          float* o_jac, float* o_lap, int64_t B, int32_t n, int32_t H,
                          int32_t d, int32_t P);

#ifdef __cplusplus
}
#endif
#endif /* FOLX_HIP_H */
