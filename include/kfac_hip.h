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
 *    tells the caller how much to bring;
 *  - the return value is 0 on success or one of the KFAC_ERR_* codes; nothing
 *    throws and nothing keeps a caller pointer after returning;
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
#define KFAC_ERR_ARG 1        /* null pointer, non-positive size, size above 2^31 elements */
#define KFAC_ERR_WORKSPACE 2  /* workspace_bytes smaller than the query says */
#define KFAC_ERR_LAUNCH 3     /* the HIP runtime refused a launch */

/* Version of this ABI (bumped when a signature changes). */
int kfac_abi_version(void);

/* ---- Kronecker factor build ------------------------------------------- */

/* Scratch needed by the three factor builders for a d x d factor reduced over
 * K terms (K = rows for Linear, n*h_out*w_out for Conv2d). */
size_t kfac_factor_workspace_bytes(int d, int64_t K);

/* C = alpha * [x,1]^T [x,1] + beta * C     (C is d x d, d = f + add_bias)
 * x is [rows, f] with row stride ldx.  The ones column is the LAST column.
 * Replaces torch.cat + torch.einsum('ki,kj->ij') + div in
 * torchsso/curv/cov/linear.py:50-59 (A, alpha = 1/n, add_bias = module has
 * bias) and :61-67 with the n^2 rescale of curvature.py:154-155,299-300
 * (G, alpha = n, add_bias = 0).  beta != 0 fuses the accumulation of
 * utils/accumulator.py:23-38 or the running average of curvature.py:185-186
 * into the GEMM epilogue; with beta == 0, C is not read. */
int kfac_factor_linear(const float* x, int64_t rows, int f, int64_t ldx, int add_bias,
                       float alpha, float beta, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

/* C = alpha * M M^T + beta * C with M = im2col(x) as [c*kh*kw (+1), n*oh*ow],
 * row order (c, kh, kw), ones ROW last; the patches are gathered tile by tile
 * into LDS and never written to memory.  x is [n, c, H, W].
 * Replaces F.unfold + transpose/reshape + cat + einsum('ik,jk->ij') + div(n) in
 * torchsso/curv/cov/conv.py:47-67 (alpha = 1/n).  groups are ignored, as there. */
int kfac_factor_conv_a(const float* x, int n, int c, int H, int W,
                       int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw,
                       int add_bias, float alpha, float beta, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

/* C = alpha * m m^T + beta * C with m = g viewed as [c, n*h*w]; g is
 * [n, c, h, w] and is read in place (no transpose copy).
 * Replaces torchsso/curv/cov/conv.py:69-74 plus the n^2 rescale of
 * curvature.py:154-155,299-300 (alpha = n / (h*w)). */
int kfac_factor_conv_g(const float* g, int n, int c, int h, int w,
                       float alpha, float beta, float* C,
                       void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KFAC_HIP_H */
