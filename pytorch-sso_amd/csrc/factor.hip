// Kronecker factor builders: symmetric products  C = alpha * P^T P + beta * C
// over the upper-triangular 128x128 tiles of C, mirrored in the epilogue.
#include "common.h"
#include "operands.h"

namespace kfac {

int choose_splits(int ntiles, long K, int* chunks_per_split) {
  const long nchunks = (K + KC - 1) / KC;
  long splits = TARGET_BLOCKS / ntiles;
  if (splits < 1) splits = 1;
  const long max_splits = nchunks / 8 > 0 ? nchunks / 8 : 1;  // >= 128 k per split
  if (splits > max_splits) splits = max_splits;
  long cps = (nchunks + splits - 1) / splits;
  if (cps < 1) cps = 1;
  splits = (nchunks + cps - 1) / cps;
  if (splits < 1) splits = 1;
  *chunks_per_split = (int)cps;
  return (int)splits;
}

template <class OP>
__global__ __launch_bounds__(NTHREADS) void syrk_kernel(OP op, int d, int K, int T, int ntiles,
                                                         int splits, int chunks_per_split,
                                                         float* C, float alpha, float beta,
                                                         float* ws) {
  __shared__ __attribute__((aligned(16))) float smem[SMEM_FLOATS];
  const int tile = blockIdx.x;
  const int split = blockIdx.y;
  int bi, bj;
  upper_tile(tile, T, bi, bj);
  const int kbeg = split * chunks_per_split * KC;
  int kend = kbeg + chunks_per_split * KC;
  if (kend > K) kend = K;
  if (splits == 1) {
    EpiStore epi{C, d, d, d, alpha, beta, bi != bj};
    gemm_tile(op, op, bi * BM, bj * BN, kbeg, kend, bi == bj, epi, smem);
  } else {
    EpiPartial epi{ws + ((size_t)split * ntiles + tile) * (BM * BN), bi * BM, bj * BN, d, d};
    gemm_tile(op, op, bi * BM, bj * BN, kbeg, kend, bi == bj, epi, smem);
  }
}

// sum the k-split partials of one tile and apply the epilogue (+ mirror)
__global__ __launch_bounds__(256) void syrk_reduce_kernel(const float* ws, int d, int T,
                                                           int ntiles, int splits, float* C,
                                                           float alpha, float beta) {
  const int tile = blockIdx.x;
  int bi, bj;
  upper_tile(tile, T, bi, bj);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = blockIdx.y * 1024 + i * 256 + threadIdx.x;
    const int row = bi * BM + (e >> 7);
    const int col = bj * BN + (e & 127);
    if (row < d && col < d) {
      float s = 0.f;
      for (int sp = 0; sp < splits; ++sp) s += ws[((size_t)sp * ntiles + tile) * (BM * BN) + e];
      const size_t idx = (size_t)row * d + col;
      float o = alpha * s;
      if (beta != 0.f) o += beta * C[idx];
      C[idx] = o;
      if (bi != bj) C[(size_t)col * d + row] = o;
    }
  }
}

template <class OP>
static int launch_syrk(const OP& op, int d, int64_t K, float alpha, float beta, float* C,
                       void* workspace, size_t workspace_bytes, hipStream_t stream) {
  const int T = cdiv(d, BM);
  const int ntiles = T * (T + 1) / 2;
  int cps;
  const int splits = choose_splits(ntiles, (long)K, &cps);
  if (splits > 1) {
    const size_t need = (size_t)splits * ntiles * BM * BN * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) return KFAC_ERR_WORKSPACE;
  }
  hipLaunchKernelGGL((syrk_kernel<OP>), dim3(ntiles, splits), dim3(NTHREADS), 0, stream, op, d,
                     (int)K, T, ntiles, splits, cps, C, alpha, beta, (float*)workspace);
  if (splits > 1) {
    hipLaunchKernelGGL(syrk_reduce_kernel, dim3(ntiles, 16), dim3(256), 0, stream,
                       (const float*)workspace, d, T, ntiles, splits, C, alpha, beta);
  }
  return launch_status();
}

}  // namespace kfac

using namespace kfac;

extern "C" {

int kfac_abi_version(void) { return 1; }

size_t kfac_factor_workspace_bytes(int d, int64_t K) {
  if (d <= 0 || K <= 0) return 0;
  const int T = cdiv(d, BM);
  const int ntiles = T * (T + 1) / 2;
  int cps;
  const int splits = choose_splits(ntiles, (long)K, &cps);
  return splits > 1 ? (size_t)splits * ntiles * BM * BN * sizeof(float) : 0;
}

int kfac_factor_linear(const float* x, int64_t rows, int f, int64_t ldx, int add_bias,
                       float alpha, float beta, float* C, void* workspace,
                       size_t workspace_bytes, void* stream) {
  if (!x || !C || rows <= 0 || f <= 0 || ldx < f) return KFAC_ERR_ARG;
  if (rows * ldx >= (int64_t)1 << 31) return KFAC_ERR_ARG;
  const int d = f + (add_bias ? 1 : 0);
  DenseKM op{x, nullptr, (int)ldx, d, add_bias ? 1 : 0};
  return launch_syrk(op, d, rows, alpha, beta, C, workspace, workspace_bytes,
                     (hipStream_t)stream);
}

int kfac_factor_conv_a(const float* x, int n, int c, int H, int W, int kh, int kw, int sh, int sw,
                       int ph, int pw, int dh, int dw, int add_bias, float alpha, float beta,
                       float* C, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !C || n <= 0 || c <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 ||
      sw <= 0 || ph < 0 || pw < 0 || dh <= 0 || dw <= 0)
    return KFAC_ERR_ARG;
  if ((int64_t)n * c * H * W >= (int64_t)1 << 31) return KFAC_ERR_ARG;
  const int OH = (H + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
  const int OW = (W + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
  if (OH <= 0 || OW <= 0) return KFAC_ERR_ARG;
  const int64_t K = (int64_t)n * OH * OW;
  if (K >= (int64_t)1 << 31) return KFAC_ERR_ARG;
  const int d = c * kh * kw + (add_bias ? 1 : 0);
  ConvA op{x, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, OH, OW, d, add_bias ? 1 : 0};
  return launch_syrk(op, d, K, alpha, beta, C, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_factor_conv_g(const float* g, int n, int c, int h, int w, float alpha, float beta,
                       float* C, void* workspace, size_t workspace_bytes, void* stream) {
  if (!g || !C || n <= 0 || c <= 0 || h <= 0 || w <= 0) return KFAC_ERR_ARG;
  if ((int64_t)n * c * h * w >= (int64_t)1 << 31) return KFAC_ERR_ARG;
  ConvG op{g, c, h * w};
  return launch_syrk(op, c, (int64_t)n * h * w, alpha, beta, C, workspace, workspace_bytes,
                     (hipStream_t)stream);
}

}  // extern "C"
