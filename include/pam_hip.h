/*
 * pam_hip.h -- C ABI of libpam_hip.so, the MI355X (gfx950) implementation of the
 * piecewise-affine arithmetic kernels of epfml/pam.
 *
 * The fourteen primitive entry points are the fourteen functions of the reference's
 * extension module (PYBIND11_MODULE in pam/cuda_kernels.cu:932-947), one to one and under
 * the same names with a pam_hip_ prefix.  Where the reference takes torch tensors and
 * returns a new one, these take raw device pointers plus sizes and element strides and
 * write into a caller-provided output.
 *
 * Conventions
 *   - every pointer is a device pointer to fp32 data on the current HIP device;
 *   - `offset` is the PAM offset as a float, 1.0f meaning none (the reference maps
 *     offset=None to 1.0, pam/cuda_bindings.py:31-32, and turns it into a bit-pattern
 *     increment, pam/cuda_kernels.cu:168);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls only
 *     enqueue work, they never synchronise, allocate or free;
 *   - return value 0 on success, negative on error; pam_hip_last_error() then returns a
 *     message for the calling thread.  Nothing is thrown.
 *   - matrices are described by (rows, cols) and element strides; any strides are
 *     accepted, and the fast paths apply when one of the two strides of an operand is 1
 *     (the row-major / column-major flags of the reference, pam/cuda_bindings.py:106-115).
 */
#ifndef PAM_HIP_H
#define PAM_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PAM_HIP_ABI_VERSION 2

enum {
    PAM_HIP_OK = 0,
    PAM_HIP_ERR_ARGUMENT = -1,   /* null pointer, negative size, size beyond 2^31 elements per dim */
    PAM_HIP_ERR_LAUNCH = -2,     /* the HIP runtime reported an error at launch */
    PAM_HIP_ERR_WORKSPACE = -3   /* workspace given but smaller than pam_hip_gemm_workspace_bytes() */
};

int pam_hip_abi_version(void);
const char *pam_hip_last_error(void);
/* Hash of the sources and flags this library was built from (pam_amd/build.py writes it in), so that a test
 * run or a benchmark can tell that the binary it loaded belongs to the tree it sits in. */
const char *pam_hip_source_hash(void);

/* Compute units and shader clock (kHz) of the current device, for roofline figures. */
int pam_hip_device_info(int *compute_units, int *clock_khz);

/* ---- elementwise, n contiguous elements (pam/cuda_kernels.cu:141-328) ------------------ */
/* C = A (*) B                         replaces pam_fwd  (elementwise_pam_caller,  :155-183) */
int pam_hip_pam_fwd(const float *a, const float *b, float *c, size_t n, float offset, void *stream);
/* dA = d/dA (A (*) B) * dC, exact     replaces pam_bwd  (elementwise_pam_bwd_caller, :200-232) */
int pam_hip_pam_bwd(const float *a, const float *b, const float *dc, float *da, size_t n, float offset, void *stream);
/* C = A (/) B                         replaces pad_fwd  (elementwise_pad_caller,  :251-279) */
int pam_hip_pad_fwd(const float *a, const float *b, float *c, size_t n, float offset, void *stream);
/* dB = d/dB (A (/) B) * dC            replaces pad_bwd  (elementwise_pad_bwd_caller, :296-328) */
int pam_hip_pad_bwd(const float *a, const float *b, const float *dc, float *db, size_t n, float offset, void *stream);

/* Both gradients of C = A (*) B or C = A (/) B in one pass over A, B, dC (20 B per element), the
 * formulas of the reference's autograd functions (pam/cuda_bindings.py:43-57, 78-97), which run two
 * to six elementwise launches for them: approx_x != 0 selects the approximate gradient of that
 * operand (product: dC (*) other; quotient: (1 (/) B) (*) dC and -((A (/) B) (/) B) (*) dC), else
 * the exact one (pam_bwd / pad_bwd above; for the quotient's dA, pam_bwd(A, 1 (/) B, dC) without offset). */
int pam_hip_pam_bwd_pair(const float *a, const float *b, const float *dc, float *da, float *db, size_t n, float offset,
                         int approx_a, int approx_b, void *stream);
int pam_hip_pad_bwd_pair(const float *a, const float *b, const float *dc, float *da, float *db, size_t n, float offset,
                         int approx_a, int approx_b, void *stream);

/* Variants of the two forward ops with one operand a single fp32 value in device memory
 * (the reference materialises broadcast scalars with flatten(), pam/cuda_kernels.cu:163-164;
 * these read 8 B/element instead of 12).  scalar_is_a != 0: C = s[0] (op) X, else C = X (op) s[0]. */
int pam_hip_pam_fwd_bcast(const float *x, const float *s, int scalar_is_a, float *c, size_t n, float offset, void *stream);
int pam_hip_pad_fwd_bcast(const float *x, const float *s, int scalar_is_a, float *c, size_t n, float offset, void *stream);

/* ---- piecewise-affine exp / log (pam/cuda_kernels.cu:334-516) -------------------------- */
/* The fp32 constant log2(base) that the four entry points below use: the double-precision logarithm rounded once
 * (the reference's kernel evaluates log2(base) per element on the device, :343, 385, 438, 481). */
float pam_hip_log2_base(float base);
/* Y = base^X  = pa_exp2(X (*) log2 base)        replaces pa_exp_fwd (:348-373) */
int pam_hip_pa_exp_fwd(const float *x, float *y, size_t n, float base, float offset, void *stream);
/*                                                replaces pa_exp_bwd (:395-423) */
int pam_hip_pa_exp_bwd(const float *x, const float *dy, float *dx, size_t n, float base, float offset, void *stream);
/* Y = log_base X = pa_log2(X) (/) log2 base     replaces pa_log_fwd (:443-468) */
int pam_hip_pa_log_fwd(const float *x, float *y, size_t n, float base, float offset, void *stream);
/*                                                replaces pa_log_bwd (:488-516) */
int pam_hip_pa_log_bwd(const float *x, const float *dy, float *dx, size_t n, float base, float offset, void *stream);

/* ---- matrix products (pam/cuda_kernels.cu:574-927) ------------------------------------- */
/* A matrix operand: pointer, batch stride, row stride, column stride (elements). */
#define PAM_HIP_MAT(name) const float *name, long name##_sb, long name##_sr, long name##_sc
#define PAM_HIP_OUT(name) float *name, long name##_sb, long name##_sr, long name##_sc

/* Scratch for a product of this shape: the words of the queues that the work-groups of a launch draw their output
 * tiles from and, for shapes with few output tiles and long k (their tiles' k ranges are cut into pieces that
 * different work-groups sum), the pieces and one arrival word per tile.  16-byte aligned.  A workspace needs no
 * preparation before its first use (any contents), every call leaves it ready for the next one, and two products
 * that overlap in time must not share one.  Passing workspace == NULL (or fewer bytes) to the calls below is
 * always valid: tiles are then never cut and every work-group computes one tile, at some cost in speed. */
size_t pam_hip_gemm_workspace_bytes(long batch, long m, long n, long k);

/* The accumulation order a product of this shape uses when the workspace is supplied.
 * k is cut into chunks of *k_chunk consecutive values (a multiple of 16; the last chunk may
 * be shorter).  Each chunk is summed in ascending k from +0 into one fp32 accumulator per
 * output, and the chunk sums are added in ascending order from +0.  One chunk (k_chunk >= k) is the
 * order of the reference kernel (pam/cuda_kernels.cu:601, 608-627), which is also the order without a
 * workspace. */
int pam_hip_gemm_plan(long batch, long m, long n, long k, int *k_chunk);

/* Y[m,n] = sum_k A[m,k] (*) B[k,n]            replaces pam_matmul_fwd (matmul_caller<&pam,false>, :703-718) */
int pam_hip_pam_matmul_fwd(const float *a, long a_sr, long a_sc, const float *b, long b_sr, long b_sc,
                           float *y, long y_sr, long y_sc, long m, long n, long k, float offset,
                           void *workspace, size_t workspace_bytes, void *stream);
/* The same product for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  What a workspace would hold goes to an
 * array of PAM_HIP_NOALLOC_SCRATCH_BYTES that the library itself holds on every GPU it runs on, for the life of
 * the process; the call allocates and frees nothing.  Results are bit-identical to pam_hip_pam_matmul_fwd with
 * a workspace of pam_hip_gemm_workspace_bytes(1, m, n, k).  A shape that needs more scratch than the array is
 * refused with PAM_HIP_ERR_WORKSPACE.  All calls on one GPU share the array: calls that overlap in time on the
 * same GPU (different streams or threads) race, so serialise them. */
#define PAM_HIP_NOALLOC_SCRATCH_BYTES (48u << 20)
int pam_hip_pam_matmul_fwd_noalloc(const float *a, long a_sr, long a_sc, const float *b, long b_sr, long b_sc,
                                   float *y, long y_sr, long y_sc, long m, long n, long k, float offset, void *stream);
/* Y = A (x) B + bias[column]: the product followed by the bias add of pam.linear
 * (pam/pam_ops.py:107-115) in one pass; the bias is added once to the finished sum (after the chunk
 * sums when k is cut), which is what the separate add computes.  bias NULL = no bias. */
int pam_hip_pam_linear_fwd(const float *a, long a_sr, long a_sc, const float *b, long b_sr, long b_sc, const float *bias,
                           float *y, long y_sr, long y_sc, long m, long n, long k, float offset,
                           void *workspace, size_t workspace_bytes, void *stream);
/* batched                                     replaces pam_bmm_fwd (matmul_caller<&pam,true>) */
int pam_hip_pam_bmm_fwd(PAM_HIP_MAT(a), PAM_HIP_MAT(b), PAM_HIP_OUT(y), long batch, long m, long n, long k,
                        float offset, void *workspace, size_t workspace_bytes, void *stream);
/* ordinary fp32 multiply through the same kernel   replaces standard_matmul / standard_bmm (:941-942) */
int pam_hip_standard_matmul(const float *a, long a_sr, long a_sc, const float *b, long b_sr, long b_sc,
                            float *y, long y_sr, long y_sc, long m, long n, long k, float ignored,
                            void *workspace, size_t workspace_bytes, void *stream);
int pam_hip_standard_bmm(PAM_HIP_MAT(a), PAM_HIP_MAT(b), PAM_HIP_OUT(y), long batch, long m, long n, long k,
                         float ignored, void *workspace, size_t workspace_bytes, void *stream);
/* Exact backward: dM[i,j] = sum_k pam_bwd(M[i,j], other, delta), where delta_l != 0 means
 * L[i,k] is the upstream gradient and R[k,j] the other forward operand, and delta_l == 0
 * the reverse.          replaces pam_matmul_bwd / pam_bmm_bwd (pam_matmul_bwd_caller, :894-924) */
int pam_hip_pam_matmul_bwd(const float *l, long l_sr, long l_sc, const float *r, long r_sr, long r_sc,
                           const float *mo, long mo_sr, long mo_sc, float *dm, long dm_sr, long dm_sc,
                           long m, long n, long k, int delta_l, float offset,
                           void *workspace, size_t workspace_bytes, void *stream);
int pam_hip_pam_bmm_bwd(PAM_HIP_MAT(l), PAM_HIP_MAT(r), PAM_HIP_MAT(mo), PAM_HIP_OUT(dm),
                        long batch, long m, long n, long k, int delta_l, float offset,
                        void *workspace, size_t workspace_bytes, void *stream);

/* ---- row-wise compositions as single kernels (pam/pam_ops.py:288-378) ------------------- */
/* The reference builds these from five to fifteen elementwise launches; the entry points
 * below compute, element for element, the same chain of primitive calls in one sweep over
 * x[rows][n] (contiguous rows, the reduced dimension last).  The order of each row sum,
 * which the reference leaves to torch.sum, is fixed: lane l of 64 adds the elements
 * l, l + 64, ... in ascending order from +0, then p[l] = p[l] + p[l ^ s] for
 * s = 32, 16, 8, 4, 2, 1. */
/* Bytes of device scratch the softmax / logsumexp entry points need (block maxima). */
size_t pam_hip_rowop_workspace_bytes(void);
/* y = softmax(x) over the last dim        replaces pam.softmax (pam/pam_ops.py:305-328):
 * x (*) log2 e with -inf kept, one global shift floor(max) written to shift[0], exp2, row
 * sum written to row_sum[rows], (/) by it. */
int pam_hip_softmax_fwd(const float *x, float *y, float *row_sum, float *shift, long rows, long n, float offset,
                        void *workspace, size_t workspace_bytes, void *stream);
/* dx for the above from the upstream gradient dy, following the autograd chain of the
 * primitives (pam/cuda_bindings.py:43-57, 78-97, 224-239).  approx_a / approx_b select the
 * approximate gradient for first / second operands of the products and quotients,
 * approx_exp the one of exp2; row_sum and shift are the forward's outputs. */
int pam_hip_softmax_bwd(const float *x, const float *dy, const float *row_sum, const float *shift, float *dx,
                        long rows, long n, float offset, int approx_a, int approx_b, int approx_exp, void *stream);
/* lse[rows] = logsumexp(x) over the last dim and/or log_softmax[rows][n] = x - lse (either
 * pointer may be NULL); the global shift goes to shift[0] if not NULL
 *                                          replaces pam.logsumexp / pam.log_softmax (:331-347) */
int pam_hip_logsumexp_fwd(const float *x, float *lse, float *log_softmax, float *shift, long rows, long n, float offset,
                          void *workspace, size_t workspace_bytes, void *stream);
/* y[rows] = sum(x[row]) (/) n             replaces pam.mean over the last dim (:288-302) */
int pam_hip_row_mean_fwd(const float *x, float *y, long rows, long n, float offset, void *stream);
/* y = layer_norm(x) over the last dim, weight and bias of n elements or NULL
 *                                          replaces pam.layer_norm (:350-378) */
int pam_hip_layer_norm_fwd(const float *x, const float *weight, const float *bias, float *y, long rows, long n,
                           float eps, float offset, void *stream);
/* Gradients of the two above, the chain autograd runs over the unfused ops
 * (pam/cuda_bindings.py:43-57, 78-97, 224-239, 262-276) in one kernel each, for rows of any length
 * (up to 1024 values a row stays in registers, longer rows are swept several times).
 * logsumexp_bwd: grad is [rows] (log_softmax == 0) or [rows][n] (the gradient of x - logsumexp(x));
 * shift is the forward's global shift.  layer_norm_bwd: dw_terms[rows][n], if not NULL, receives
 * the per-element terms whose sum over rows is the weight gradient (the bias gradient is the sum
 * of dy over rows). */
int pam_hip_logsumexp_bwd(const float *x, const float *grad, const float *shift, float *dx, long rows, long n,
                          int log_softmax, float offset, int approx_a, int approx_b, int approx_exp, void *stream);
int pam_hip_layer_norm_bwd(const float *x, const float *weight, const float *dy, float *dx, float *dw_terms, long rows, long n,
                           float eps, float offset, int approx_a, int approx_b, int approx_exp, void *stream);

/* ---- convolution without the unfolded matrix (pam/pam_ops.py:118-160) ---------------------- */
/* The reference computes conv2d as unfold -> transpose copy -> PAM linear, a kh*kw-fold copy of
 * the input.  These entry points run the same products and sums on the matrix kernel with the
 * image patches read in place: x[batch][c][h][w] and w[co][c][kh][kw] contiguous, dilation 1,
 * output size (in + 2 pad - k) / stride + 1.  groups > 1 is the grouped convolution of
 * pam.conv2d_group (:163-198): w[co][c / groups][kh][kw], channels and filters fall into groups that
 * do not mix (groups = 1 otherwise); one launch covers all (image, group) pairs, with one copy of the
 * weights per image in the workspace where a product reads them -- unless those copies would exceed
 * 32 MiB, then one launch per group; depthwise convolutions (groups = c = co, kh*kw < 128) have kernels
 * of their own that give the same sums in the same order.  Sums run over k = (c, i, j) of the group in ascending order in
 * the chunks pam_hip_gemm_plan(batch * groups, co / groups, ho*wo, (c / groups)*kh*kw) reports
 * (batch in place of batch * groups for a product that is launched per group). */
size_t pam_hip_conv2d_workspace_bytes(long batch, long c, long h, long w, long co, long kh, long kw,
                                      long stride_h, long stride_w, long pad_h, long pad_w, long groups, int which, float offset);
/* which: 0 forward, 1 weight gradient, 2 input gradient */
/* y[batch][co][ho][wo] = sum_k x_patch (*) (w (*) offset)           replaces pam.conv2d's forward */
int pam_hip_conv2d_fwd(const float *x, const float *w, float *y, long batch, long c, long h, long wd, long co, long kh, long kw,
                       long stride_h, long stride_w, long pad_h, long pad_w, long groups, float offset,
                       void *workspace, size_t workspace_bytes, void *stream);
/* dw[batch][co][c*kh*kw]: each image's contribution to the weight gradient (the caller sums over
 * the batch, as autograd does for the reference's broadcast weight).  exact == 0: the
 * approximate gradient sum_l x_patch (*) (dy (*) offset) (pam/cuda_bindings.py:160-161);
 * exact != 0: sum_l pam_bwd(w, x_patch, dy) (:162-164), w required. */
int pam_hip_conv2d_bwd_weight(const float *x, const float *dy, const float *w, float *dw, long batch, long c, long h, long wd,
                              long co, long kh, long kw, long stride_h, long stride_w, long pad_h, long pad_w, long groups,
                              int exact, float offset, void *workspace, size_t workspace_bytes, void *stream);

/* dx[batch][c][h][w] for stride 1 (any other stride is an argument error: the caller keeps the
 * unfolded path) and pad <= k - 1: the gradient of the input is the convolution of dy, padded by
 * k - 1 - pad, with the weights flipped and their channel indices exchanged, so it runs on the same
 * kernel with dy's patches read in place instead of through the [c*kh*kw, ho*wo] gradient of the
 * unfolded matrix and its overlap-add.  exact == 0: sum_k (w (*) offset) (*) dy_patch
 * (pam/cuda_bindings.py:157-158); exact != 0: sum_k pam_bwd(x, w, dy_patch) (:158-159), x required
 * (one x per output element: every patch entry that an input pixel fills is that pixel).
 * Sums run over k = (co, i, j) ascending in the chunks pam_hip_gemm_plan(batch, c, h*w, co*kh*kw)
 * reports; the reference's order is that of its matrix kernel followed by torch's fold. */
int pam_hip_conv2d_bwd_input(const float *dy, const float *w, const float *x, float *dx, long batch, long c, long h, long wd,
                             long co, long kh, long kw, long stride_h, long stride_w, long pad_h, long pad_w, long groups,
                             int exact, float offset, void *workspace, size_t workspace_bytes, void *stream);

/* ---- power with a scalar exponent ---------------------------------------------------------- */
/* y = x ** exponent = pa_exp2(pa_log2(x) (*) exponent), 0 where x is 0: the three elementwise
 * launches and the select of pam.pow (pam/pam_ops.py:70-79) in one pass.  pow_bwd: the gradient for
 * x that autograd chains through them (pam/cuda_bindings.py:43-57, 224-239, 262-276); approx_a
 * selects the approximate gradient of the product, approx_exp that of exp2 and log2. */
int pam_hip_pow_fwd(const float *x, float *y, size_t n, float exponent, float offset, void *stream);
int pam_hip_pow_bwd(const float *x, const float *dy, float *dx, size_t n, float exponent, float offset,
                    int approx_a, int approx_exp, void *stream);

/* ---- optimizer step ---------------------------------------------------------------------- */
/* One Adam update of n parameters in place, every product, the quotient and the square root
 * a PAM op                replaces the op-table arithmetic of the training recipe's optimizer
 * (submodules/fairseq/fairseq/optim/adam.py:226-252 in the reference tree):
 *   m = m (*) beta1 + g (*) (1 - beta1);   v = v (*) beta2;   v += (g (*) g) (*) (1 - beta2)
 *   denom = pow(v, 0.5) + eps;   if has_decay: p -= p (*) decay;   p -= (m (/) denom) (*) step_size
 * The scalars are the fp32 roundings of the host's double-precision values (decay = weight
 * decay x learning rate, step_size = lr sqrt(1 - beta2^t) / (1 - beta1^t)). */
int pam_hip_adam_step(float *p, const float *g, float *m, float *v, size_t n, float beta1, float one_minus_beta1,
                      float beta2, float one_minus_beta2, float eps, float decay, int has_decay, float step_size,
                      float offset, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PAM_HIP_H */
