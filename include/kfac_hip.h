/* C ABI of the MI355X (gfx950) K-FAC curvature engine: libkfac_hip.so.
 *
 * The reference (cybertronai/pytorch-sso) has no native boundary: its hot path
 * is torch / CuPy calls made from Python.  Each entry point below replaces the
 * arithmetic of one such call site (cited as file:line of the reference) and
 * is what the Python classes of the same names bind through ctypes.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer to contiguous row-major fp32 unless the
 *    comment says "host";
 *  - `stream` is a hipStream_t passed as void*; all work is enqueued on it and
 *    nothing synchronises with the host;
 *  - no entry point allocates or frees memory; scratch comes in as
 *    (workspace, workspace_bytes) and the matching *_workspace_bytes() query
 *    tells the caller how much to bring (one entry point,
 *    kfac_damped_inverse_batched_static, brings its own fixed scratch instead);
 *  - the return value is 0 on success or one of the KFAC_ERR_* codes; nothing
 *    throws and nothing keeps a caller pointer after returning;
 *  - sizes: any single matrix (factor, inverse, gradient viewed as 2-D) is at most
 *    1 GiB (16384 x 16384 fp32); layer inputs of any size are accepted (the factor
 *    builders consume them in slices of at most 1 GiB along the batch dimension);
 *  - entry points are re-entrant: they may be called from any host thread
 *    (the backward hooks of the host code run on autograd's worker thread).
 */
#ifndef KFAC_HIP_H
#define KFAC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KFAC_OK 0
#define KFAC_ERR_ARG 1        /* null pointer, non-positive size, matrix above 16384 x 16384 */
#define KFAC_ERR_WORKSPACE 2  /* workspace_bytes smaller than the query says */
#define KFAC_ERR_LAUNCH 3     /* the HIP runtime refused a launch */
#define KFAC_ERR_TOO_LARGE 4  /* the problem does not fit the library's built-in scratch */

/* Version of this ABI (bumped when a signature changes). */
int kfac_abi_version(void);

/* ---- Kronecker factor build ------------------------------------------- */

/* Scratch needed by the three factor builders for a d x d factor reduced over
 * K terms (K = rows for Linear, n*h_out*w_out for Conv2d). */
size_t kfac_factor_workspace_bytes(int d, int64_t K);

/* C = alpha * [x,1]^T [x,1] + beta * C_prev     (C is d x d, d = f + add_bias;
 * C_prev == NULL: the old contents of C; a C_prev different from C lets the
 * running average be written into a second buffer while C_prev stays intact)
 * x is [rows, f] with row stride ldx.  The ones column is the LAST column.
 * Replaces torch.cat + torch.einsum('ki,kj->ij') + div in
 * torchsso/curv/cov/linear.py:50-59 (A, alpha = 1/n, add_bias = module has
 * bias) and :61-67 with the n^2 rescale of curvature.py:154-155,299-300
 * (G, alpha = n, add_bias = 0).  beta != 0 fuses the accumulation of
 * utils/accumulator.py:23-38 or the running average of curvature.py:185-186
 * into the GEMM epilogue; with beta == 0, neither C nor C_prev is read.  C_prev
 * must be symmetric (what these routines write is, to the bit): its upper
 * triangle is read, its lower one only inside the 32x32 blocks on the diagonal,
 * and C is written symmetric (the blocks below the diagonal are mirror images
 * of those above); a C_prev that is not symmetric gives neither the
 * element-wise average nor a symmetric one. */
int kfac_factor_linear(const float* x, int64_t rows, int f, int64_t ldx, int add_bias,
                       float alpha, float beta, const float* C_prev, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Scratch needed by kfac_factor_conv_a for this geometry (it may exceed
 * kfac_factor_workspace_bytes of the same factor). */
size_t kfac_factor_conv_a_workspace_bytes(int n, int c, int H, int W, int kh, int kw,
                                          int sh, int sw, int ph, int pw, int dh, int dw,
                                          int add_bias);

/* C = alpha * M M^T + beta * C_prev with M = im2col(x) as [c*kh*kw (+1), n*oh*ow],
 * row order (c, kh, kw), ones ROW last; M is never written to memory.
 * x is [n, c, H, W].  Two kernels, same result: in general the patches are
 * gathered tile by tile into LDS; for a stride-1, bias-free layer with 2..9
 * kernel taps the blocks of C that share a tap displacement are built from one
 * spatial correlation of the input with itself (3.4x fewer flops for 3x3).
 * Replaces F.unfold + transpose/reshape + cat + einsum('ik,jk->ij') + div(n) in
 * torchsso/curv/cov/conv.py:47-67 (alpha = 1/n).  groups are ignored, as there. */
int kfac_factor_conv_a(const float* x, int n, int c, int H, int W,
                       int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw,
                       int add_bias, float alpha, float beta, const float* C_prev, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Plan queries (no device needed): the fp32 MFMA flops the factor builders execute for a
 * d x d factor reduced over K terms (kfac_factor_linear, kfac_factor_conv_g and the
 * pointwise case of kfac_factor_conv_a) and for a Conv2d input factor of the given
 * geometry: whole tiles of the upper triangle, whole reduction chunks, the shared spatial
 * correlations of a stride-1 k x k layer.  For utilisation figures next to the
 * algorithmic 2*d*d*K. */
double kfac_factor_executed_flops(int d, int64_t K);
double kfac_factor_conv_a_executed_flops(int n, int c, int H, int W, int kh, int kw,
                                         int sh, int sw, int ph, int pw, int dh, int dw,
                                         int add_bias);

/* C = alpha * m m^T + beta * C_prev with m = g viewed as [c, n*h*w]; g is
 * [n, c, h, w] and is read in place (no transpose copy).
 * Replaces torchsso/curv/cov/conv.py:69-74 plus the n^2 rescale of
 * curvature.py:154-155,299-300 (alpha = n / (h*w)). */
int kfac_factor_conv_g(const float* g, int n, int c, int h, int w,
                       float alpha, float beta, const float* C_prev, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

/* ---- Grouped factor build (the products of many layers in one call) ------ */

#define KFAC_FACTOR_LINEAR 0   /* kfac_factor_linear: x is [rows, c], ldx = c */
#define KFAC_FACTOR_CONV_A 1   /* kfac_factor_conv_a: x is [rows, c, H, W] */
#define KFAC_FACTOR_CONV_G 2   /* kfac_factor_conv_g: x is [rows, c, H, W] (H, W of the output) */

/* One product of a grouped call: the arguments of the single-product entry point of
 * its `kind` (fields that kind does not use are ignored). */
typedef struct kfac_factor_job {
  int kind;
  int add_bias;
  const float* x;            /* device */
  int64_t rows;              /* linear: rows of x; conv: batch size n */
  int c, H, W;
  int kh, kw, sh, sw, ph, pw, dh, dw;     /* KFAC_FACTOR_CONV_A only */
  float alpha, beta;
  const float* C_prev;       /* device, may be NULL (see kfac_factor_linear) */
  float* C;                  /* device */
} kfac_factor_job;

/* Scratch for kfac_factor_grouped on this list (`jobs` is a HOST array): the device
 * tables of its launches, the k-split partials of all products at once, the zero-padded
 * copies of the inputs of strided / padded k x k convolutions (about 1.5 x such an input
 * for a 3x3 kernel of stride 2), and the scratch of the products that go through their
 * single-product routine. */
size_t kfac_factor_grouped_workspace_bytes(int count, const kfac_factor_job* jobs);

/* Every product of the list, C_i = alpha_i * P_i^T P_i + beta_i * C_prev_i, with the same
 * results as `count` calls of kfac_factor_linear / kfac_factor_conv_a / kfac_factor_conv_g
 * up to the summation order of the k-splits, in a handful of launches: one per operand
 * kind and tile size holds the (tile, k-split) work items of all its products, longest
 * first, and two more reduce the partial sums of all of them.  For a host that collects
 * the factor products of a whole forward / backward pass (hooks of
 * torchsso/curv/curvature.py:118-155 calling cov/linear.py:50-67 and cov/conv.py:47-74
 * layer by layer) and hands them over before the first reader of a factor: a launch per
 * layer drains and refills the chip a hundred times per step.  The outputs C_i must be
 * distinct buffers, and no C_i may be an input or C_prev of another product of the call.
 * Stride-1 k x k convolution inputs go through the correlation kernels (all such layers
 * of the call in one launch each); inputs above 1 GiB run through their single-product
 * routines on the same stream. */
int kfac_factor_grouped(int count, const kfac_factor_job* jobs, void* workspace,
                        size_t workspace_bytes, void* stream);

/* Plan query: the fp32 MFMA flops kfac_factor_grouped executes for this list. */
double kfac_factor_grouped_executed_flops(int count, const kfac_factor_job* jobs);

/* ---- Damped factor inversion ------------------------------------------- */

/* Scratch for the three batched routines below: a descriptor table plus one
 * n x n buffer per matrix.  `dims` is a HOST array of `count` sizes. */
size_t kfac_inverse_workspace_bytes(int count, const int* dims);

/* Plan query: the fp32 MFMA flops the batched inversion executes for matrices of these
 * sizes (HOST arrays): blocked Cholesky (diagonal blocks, row panels, trailing updates
 * with whole diagonal tiles), the triangular inverse, and Y Y^T for the matrices whose
 * explicit inverse is formed (factored[i] == 0, or factored == NULL). */
double kfac_inverse_executed_flops(int count, const int* dims, const int* factored);

/* For every layer l:  pi = sqrt((tr A/dA) / (tr G/dG)), r = sqrt(damping[l]),
 *   Ainv = (A + r*pi*I)^-1 ,  Ginv = (G + (r/pi)*I)^-1 .
 * The traces, pi and the diagonal shift are computed on the device and the
 * shift is added while the factor is copied into the Cholesky work area; all
 * 2*layers matrices are factored, triangular-inverted and multiplied back in
 * one shared launch sequence (blocked Cholesky, 128-wide panels).
 * Replaces KronCurvature.update_inv, torchsso/curv/curvature.py:302-312, with
 * add_value_to_diagonal :334-340 and torchsso.utils.inv,
 * utils/inv_cupy.py:27-34 (cuSOLVER potrf + potrs against I, :114-128).
 * dA, dG, damping and the four pointer arrays are HOST arrays of length
 * `layers` (the pointers in them are device pointers; A and G are only read;
 * Ainv/Ginv must not alias A/G).  damping[l] is the layer's damping + l2_reg_ema
 * (curvature.py:102-104).  info is a DEVICE array of 2*layers ints: info[2l]
 * for A_l, info[2l+1] for G_l; 0 = success, k > 0 = the leading minor of order
 * k is not positive definite (the reference never reads cuSOLVER's dev_info,
 * inv_cupy.py:124,130). */
int kfac_pi_damped_inverse_batched(int layers, const int* dA, const int* dG,
                                   const float* const* A, const float* const* G,
                                   const float* damping,
                                   float* const* Ainv, float* const* Ginv, int* info,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* kfac_pi_damped_inverse_batched that also delivers, for every matrix whose Astd[l] / Gstd[l]
 * is non-NULL, the upper Cholesky factor of its inverse:
 *   Astd[l]^T Astd[l] = Ainv[l],  Gstd[l]^T Gstd[l] = Ginv[l],  upper triangular, zero below.
 * Replaces KronCurvature.update_inv followed by update_std, torchsso/curv/curvature.py:302-312
 * and :317-321 (torchsso.utils.cholesky of each inverse, utils/cholesky_cupy.py:9-14), without
 * the second factorisation: such a layer's damped factors are factored back to front (rows and
 * columns reversed, J X J = R^T R), so that X^-1 = J R^-1 R^-T J = W^T W with W = J R^-T J upper
 * triangular with a positive diagonal -- the Cholesky factor the reference computes from the
 * inverse -- and W is read off the triangular inverse the inversion forms anyway.  For these
 * matrices a non-zero info[] counts the failing leading minor of the REVERSED matrix. */
int kfac_pi_damped_inverse_std_batched(int layers, const int* dA, const int* dG,
                                       const float* const* A, const float* const* G,
                                       const float* damping,
                                       float* const* Ainv, float* const* Ginv,
                                       float* const* Astd, float* const* Gstd, int* info,
                                       void* workspace, size_t workspace_bytes, void* stream);

/* kfac_pi_damped_inverse_batched for a caller that applies the inverses rather than reads
 * them: per matrix EXACTLY ONE of Ainv[l] / Afac[l] (and of Ginv[l] / Gfac[l]) is non-NULL.
 * Where the `fac` pointer is given the result is the triangular factor of the inverse,
 *   Afac[l] Afac[l]^T = (A + r*pi*I)^-1 ,  Gfac[l] Gfac[l]^T = (G + (r/pi)*I)^-1 ,
 * upper triangular with zeros below the diagonal (the inverse of the Cholesky factor), and the
 * explicit inverse, the last third of that matrix's inversion work, is never formed:
 * kfac_precondition_factored_batched applies the factor twice at the cost of applying the
 * inverse once.  Replaces KronCurvature.update_inv, torchsso/curv/curvature.py:302-312 with
 * utils/inv_cupy.py:27-34; the explicit inverse of a factored matrix is fac * fac^T.
 * pi, r, info and the workspace as for kfac_pi_damped_inverse_batched. */
int kfac_pi_damped_inverse_factored_batched(int layers, const int* dA, const int* dG,
                                            const float* const* A, const float* const* G,
                                            const float* damping,
                                            float* const* Ainv, float* const* Ginv,
                                            float* const* Afac, float* const* Gfac, int* info,
                                            void* workspace, size_t workspace_bytes, void* stream);

/* dst[i] = (src[i] + damp[i]*I)^-1 for `count` symmetric positive definite
 * matrices of sizes dims[i]; damp may be NULL (no shift).  Host arrays as
 * above; info is a DEVICE array of `count` ints.
 * Replaces Curvature._inv, curvature.py:197-200, and torchsso.utils.inv. */
int kfac_damped_inverse_batched(int count, const int* dims, const float* const* src,
                                const float* damp, float* const* dst, int* info,
                                void* workspace, size_t workspace_bytes, void* stream);

/* kfac_damped_inverse_batched for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid it).  It has no
 * counterpart in the reference.  Same arguments and results as kfac_damped_inverse_batched
 * without the workspace: the descriptor table and the n x n buffers live in an array that
 * is part of the library's code object (kfac_static_workspace_bytes() = 8 MiB, held by
 * every GPU the library runs on until the process ends), and the call makes no hipMalloc,
 * hipFree or other allocating call.  A list that needs more than that
 * (kfac_inverse_workspace_bytes(count, dims) > kfac_static_workspace_bytes(); e.g. one
 * matrix above 1448 x 1448) is rejected with KFAC_ERR_TOO_LARGE before anything is
 * launched.  The first call on a device looks up the array's address on that device,
 * creates the event below (and raises the LDS limit of the kernels); make that call outside
 * a capture.  All calls on one GPU share the array; they are put in order: a call's stream
 * first waits for an event that the previous call on that GPU recorded behind its last
 * kernel, so calls on two streams or from two threads run one after the other instead of
 * racing.  A stream under graph capture takes no part in that (inside a graph the graph's
 * own order applies): calls captured into graphs that may run at the same time still
 * race. */
size_t kfac_static_workspace_bytes(void);
int kfac_damped_inverse_batched_static(int count, const int* dims, const float* const* src,
                                       const float* damp, float* const* dst, int* info,
                                       void* stream);

/* dst[i] = U with src[i] = U^T U, U upper triangular (strictly lower part
 * written as zero).  Replaces torchsso.utils.cholesky(m, upper=True),
 * utils/cholesky_cupy.py:9-14, as used by KronCurvature.update_std,
 * curvature.py:317-321. */
int kfac_cholesky_upper_batched(int count, const int* dims, const float* const* src,
                                float* const* dst, int* info,
                                void* workspace, size_t workspace_bytes, void* stream);

/* ---- Preconditioning and posterior sampling ---------------------------- */

/* Scratch for the two routines below (dG, dA: HOST arrays). */
size_t kfac_precondition_workspace_bytes(int layers, const int* dG, const int* dA);

/* Plan query: the fp32 MFMA flops the preconditioning of these layers executes (HOST
 * arrays; a NULL flag array: no side is given by its triangular factor): whole 128 x 128
 * tiles; a triangular operand is applied twice, each time over the non-zero part of the
 * reduction (the diagonal tiles' zero half included). */
double kfac_precondition_executed_flops(int layers, const int* dG, const int* dA,
                                        const int* g_factored, const int* a_factored);

/* For every layer:  [gradW | gradb] <- Ginv * [gradW | gradb] * Ainv, in place.
 * gradW is [dG, dA - 1] when gradb[l] != NULL (dA counts the bias column,
 * which is LAST) and [dG, dA] otherwise; for Conv2d gradW is the weight
 * gradient viewed as [c_out, c_in*kh*kw].  Two chained MFMA products per
 * launch pair for the whole layer set; no concatenated copy is made.
 * Replaces torch.cat + G_inv.mm(grad).mm(A_inv) + copy_ in
 * torchsso/curv/cov/linear.py:69-84 and cov/conv.py:76-92.
 * All array arguments are HOST arrays of length `layers`. */
int kfac_precondition_batched(int layers, const int* dG, const int* dA,
                              const float* const* Ginv, const float* const* Ainv,
                              float* const* gradW, float* const* gradb,
                              void* workspace, size_t workspace_bytes, void* stream);

/* kfac_precondition_batched with some or all inverses given by their triangular factors, as
 * kfac_pi_damped_inverse_factored_batched delivers them: Gop[l] is the upper-triangular Gfac
 * (Gfac Gfac^T = Ginv, zeros below the diagonal) where g_factored[l] != 0, else Ginv itself;
 * Aop[l] and a_factored[l] likewise (a NULL flag array means "all factored").
 *   [gradW | gradb] <- Gfac (Gfac^T [gradW | gradb] Afac) Afac^T , in place;
 * a factored side takes two products that each skip the zero half of the triangular operand,
 * which together cost what the one dense product with the explicit inverse costs.  Replaces
 * the same call sites, torchsso/curv/cov/linear.py:69-84 and cov/conv.py:76-92. */
size_t kfac_precondition_factored_workspace_bytes(int layers, const int* dG, const int* dA);
int kfac_precondition_factored_batched(int layers, const int* dG, const int* dA,
                                       const float* const* Gop, const float* const* Aop,
                                       const int* g_factored, const int* a_factored,
                                       float* const* gradW, float* const* gradb,
                                       void* workspace, size_t workspace_bytes, void* stream);

/* For every layer:  [paramW | paramb] = [meanW | meanb] + std_scale * U_G * E * U_A
 * with U_G, U_A the upper Cholesky factors of the inverses and E = noise[l], a
 * [dG, dA] standard-normal matrix drawn by the caller (so that the random
 * stream stays the host framework's).  Replaces
 * torchsso/curv/cov/linear.py:86-100 and cov/conv.py:94-108. */
int kfac_sample_batched(int layers, const int* dG, const int* dA,
                        const float* const* U_G, const float* const* U_A,
                        const float* const* noise,
                        const float* const* meanW, const float* const* meanb,
                        float* const* paramW, float* const* paramb, float std_scale,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ---- HBM-bound tails (one launch per tensor list) ----------------------- */

/* Scratch for the four *_batched routines below. */
size_t kfac_vector_workspace_bytes(int count);

/* y[i] = a * x[i] + b * y[i]  (b == 0: y is not read).
 * Running average of curvature.py:185-186 (a = ema_decay, b = 1 - ema_decay,
 * x = data, y = ema), accumulation of utils/accumulator.py:23-38 (b = 1) and
 * the l2 term grad += l2_reg * param of optim/secondorder.py:238-243. */
int kfac_axpby_batched(int count, const int64_t* numel, const float* const* x,
                       float* const* y, float a, float b,
                       void* workspace, size_t workspace_bytes, void* stream);

/* inv[i] = 1 / ((use_sqrt ? sqrt(ema[i]) : ema[i]) + damping[i])
 * DiagCurvature._inv, curvature.py:226-232. */
int kfac_diag_inverse_batched(int count, const int64_t* numel, const float* const* ema,
                              float* const* inv, const float* damping, int use_sqrt,
                              void* workspace, size_t workspace_bytes, void* stream);

/* grad[i] *= inv[i]   DiagCurvature.precondition_grad, curvature.py:234-238. */
int kfac_diag_precondition_batched(int count, const int64_t* numel, const float* const* inv,
                                   float* const* grad,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* Diagonal covariance of a Linear layer: W[i][j] = alpha * sum_b g[b][i]^2 a[b][j]^2
 * ([fout, fin]) and, with add_bias, bvec[i] = alpha * sum_b g[b][i]^2.
 * g is [n, fout], a is [n, fin].  Replaces the two element-wise squares, the
 * einsum('ki,kj->ij') and the mean of torchsso/curv/cov/linear.py:28-45 with
 * the n^2 rescale of curvature.py:154-158 folded in (alpha = n). */
int kfac_diag_cov_linear(const float* g, const float* a, int n, int fout, int fin, int add_bias,
                         float alpha, float* W, float* bvec, void* stream);

/* Diagonal covariance of a Conv2d weight:
 *   out[i][j] = alpha * sum_b (sum_k g[b][i][k] * M_b[j][k])^2     ([cout, c*kh*kw])
 * with M_b = im2col of sample b, i.e. the batch sum of the squared per-sample
 * weight gradients.  g is [n, cout, OH, OW], x is [n, c, H, W].
 * Replaces F.unfold + einsum('bik,bjk->bij') + mul + mean of
 * torchsso/curv/cov/conv.py:15-36 (alpha = n after the n^2 rescale); neither the
 * unfolded input nor the per-sample gradients are written to memory. */
size_t kfac_diag_cov_conv2d_workspace_bytes(int n, int cout, int c, int kh, int kw);
int kfac_diag_cov_conv2d(const float* g, const float* x, int n, int cout, int c, int H, int W,
                         int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw,
                         float alpha, float* out,
                         void* workspace, size_t workspace_bytes, void* stream);

/* y[i] = sqrt(x[i])   std of a diagonal curvature, curvature.py:240-241. */
int kfac_sqrt_batched(int count, const int64_t* numel, const float* const* x, float* const* y,
                      void* workspace, size_t workspace_bytes, void* stream);

/* y[i] = max(x[i], y[i])   running maximum of the average, curvature.py:189-191. */
int kfac_max_batched(int count, const int64_t* numel, const float* const* x, float* const* y,
                     void* workspace, size_t workspace_bytes, void* stream);

/* param = mean + std_scale * noise * std, element-wise; noise_to_param[i] holds the
 * standard-normal noise on entry and the sampled parameter on return.
 * DiagCurvature.sample_params, curvature.py:243-246 (std_scale is a HOST array). */
int kfac_diag_sample_batched(int count, const int64_t* numel, const float* const* mean,
                             const float* const* std_dev, float* const* noise_to_param,
                             const float* std_scale,
                             void* workspace, size_t workspace_bytes, void* stream);

/* g += weight_decay*p ; if momentum: buf = momentum*buf + g, g = buf ; p -= lr*g
 * with g written back, per tensor i with its own lr/momentum/weight_decay
 * (HOST arrays).  The preconditioned-gradient tail of
 * SecondOrderOptimizer.update_preprocess / update,
 * optim/secondorder.py:248-261 and :225-231. */
int kfac_sgd_update_batched(int count, const int64_t* numel, float* const* param,
                            float* const* grad, float* const* momentum_buf,
                            const float* lr, const float* momentum, const float* weight_decay,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---- Fisher weighting ---------------------------------------------------- */

/* out[r][i] = x[r][i] * (use_sqrt ? sqrt(w[r]) : w[r]) for `rows` rows of `len`
 * contiguous elements (out may equal x).  The true-Fisher curvatures weigh each
 * sample's output gradient by a probability: G = sum_n prob[n] g_n g_n^T
 * (torchsso/curv/fisher/linear.py:47-54, fisher/conv.py:61-70 of the reference,
 * pg = g * prob then einsum(pg, g)).  With use_sqrt the weighted gradient
 * sqrt(prob) * g can go through the symmetric factor kernels unchanged, and the
 * sum over classes / MC samples (Fisher.accumulate_cov, fisher/__init__.py:24-28)
 * is their beta = 1 epilogue.  Without it: prob * (sum_hw g^2) of
 * fisher/batchnorm.py:18-21. */
int kfac_scale_rows(const float* x, const float* w, int64_t rows, int64_t len, int use_sqrt,
                    float* out, void* stream);

/* ---- BatchNorm diagonal curvature -------------------------------------- */

/* out[row] = sum_i ((x[row*len + i] - shift[c]) / scale[c])^2, c = row % channels;
 * scale/shift may be NULL.  With x = the BatchNorm output and scale/shift its
 * weight/bias this is sum_hw x_hat^2 of cov/batchnorm.py:36-37 without
 * materialising x_hat (curvature.py:123-134); with NULLs on grad_output it is
 * sum_hw g^2 (:38). */
int kfac_rowsq_sum(const float* x, int64_t rows, int channels, int len,
                   const float* scale, const float* shift, float* out, void* stream);

/* w_curv[c] = alpha * sum_n sx[n][c]*sg[n][c] ; b_curv[c] = alpha * sum_n sg[n][c]
 * (b_curv may be NULL).  cov/batchnorm.py:40-49 with alpha = n^2 / n from the
 * rescale of curvature.py:154-158. */
int kfac_bn_diag_combine(const float* sx, const float* sg, int n, int channels, float alpha,
                         float* w_curv, float* b_curv, void* stream);

/* The backward half of the BatchNorm diagonal curvature in one call:
 *   w_curv[c] = alpha * sum_n sx[n][c] * (sum_hw g[n][c][hw]^2),
 *   b_curv[c] = alpha * sum_n (sum_hw g[n][c][hw]^2)            (b_curv may be NULL),
 * i.e. kfac_rowsq_sum on grad_output followed by kfac_bn_diag_combine
 * (cov/batchnorm.py:38-49, alpha as above).  For rows of up to 1024 elements one launch
 * does both and the row sums never reach memory; longer rows take the two kernels and
 * need kfac_bn_diag_cov_workspace_bytes(n, channels) bytes of workspace (the short-row
 * path ignores it). */
size_t kfac_bn_diag_cov_workspace_bytes(int n, int channels);
int kfac_bn_diag_cov(const float* g, int n, int channels, int len, const float* sx, float alpha,
                     float* w_curv, float* b_curv, void* workspace, size_t workspace_bytes,
                     void* stream);

/* kfac_bn_diag_cov for the BatchNorm layers of a whole backward pass in ONE launch (HOST arrays
 * of length `count`; b_curv may be NULL, or hold NULLs): a workgroup takes one channel of
 * one layer, so the small layers at the end of a network (a few MB each, a launch of their
 * own lasts as long as its latency) share the chip with the large ones.  Same formulas,
 * cov/batchnorm.py:38-49 with the rescale of curvature.py:154-158; n[i] <= 2048. */
size_t kfac_bn_diag_cov_batched_workspace_bytes(int count);
int kfac_bn_diag_cov_batched(int count, const float* const* g, const int* n, const int* channels,
                             const int* len, const float* const* sx, const float* alpha,
                             float* const* w_curv, float* const* b_curv, void* workspace,
                             size_t workspace_bytes, void* stream);

/* ---- Wire format: triangular packing ------------------------------------ */

/* The reference ships factors between ranks as one flat fp32 buffer: arrays back
 * to back, a symmetric matrix as its upper triangle row by row (element (y, x),
 * x >= y, at n*y - y*(y+1)/2 + x -- what cuBLAS strttp(FILL_MODE_LOWER) makes of
 * the row-major array), anything else whole.  Replaces Packer.pack / unpack and
 * the 'unpack' element-wise kernel of
 * torchsso/utils/chainer_communicators/_utility.py:16-104.  Per array i (HOST
 * arrays): numel[i] elements; triangular[i] != 0: a dims[i] x dims[i] matrix
 * (numel[i] == dims[i]^2).  The list starts at buffer + offset (in elements);
 * kfac_packed_numel gives its length.  unpack fills both triangles. */
size_t kfac_pack_workspace_bytes(int count);
int64_t kfac_packed_numel(int count, const int64_t* numel, const int* dims,
                          const int* triangular);
int kfac_pack_batched(int count, const float* const* arrays, const int64_t* numel,
                      const int* dims, const int* triangular, float* buffer, int64_t offset,
                      void* workspace, size_t workspace_bytes, void* stream);
int kfac_unpack_batched(int count, float* const* arrays, const int64_t* numel,
                        const int* dims, const int* triangular, const float* buffer,
                        int64_t offset, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KFAC_HIP_H */
