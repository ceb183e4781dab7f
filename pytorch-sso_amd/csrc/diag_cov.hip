// Diagonal (element-wise) covariance of Linear and Conv2d layers: the mean over
// the batch of the squared per-sample gradients.
//
//   Linear:  per-sample gradient g_b a_b^T, so  D[i][j] = sum_b g[b][i]^2 a[b][j]^2,
//            one product of the squared operands (squared on the way into LDS);
//   Conv2d:  per-sample gradient W_b = g_b M_b^T (M_b = im2col of sample b), so
//            D[i][j] = sum_b (sum_k g_b[i][k] M_b[j][k])^2: a workgroup keeps one
//            output tile, runs the implicit-im2col product once per sample and
//            adds the squares of its accumulators to a second set of registers.
//            Neither the unfolded input nor the [n, c_out, c_in*kh*kw] tensor of
//            per-sample gradients is ever written to memory.
#include "common.h"
#include "operands.h"

namespace kfac {

struct SqDenseKM : DenseKM {
  static constexpr bool square = true;
};

// weight part to W[M][fin], the extra column (bias) to bvec[M]
struct EpiWeightBias {
  float* W;
  float* bvec;
  int M, N, fin;
  float alpha;
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < M && col < N) {
      if (col < fin)
        W[(size_t)row * fin + col] = alpha * v;
      else
        bvec[row] = alpha * v;
    }
  }
};

__global__ __launch_bounds__(NTHREADS, 3) void diag_linear_kernel(const float* g, const float* a,
                                                                  int n, int fout, int fin,
                                                                  int add_bias, float alpha,
                                                                  float* W, float* bvec) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int N = fin + (add_bias ? 1 : 0);
  SqDenseKM P{{g, nullptr, fout, fout, 0}};
  SqDenseKM Q{{a, nullptr, fin, N, add_bias ? 1 : 0}};
  EpiWeightBias epi{W, bvec, fout, N, fin, alpha};
  gemm_tile(P, Q, blockIdx.y * BM, blockIdx.x * BN, 0, n, false, epi, smem);
}

// sum of squares of the accumulators over the calls of the tile engine
struct EpiSquares {
  static constexpr bool indexed = true;
  float sq[64];
  __device__ __forceinline__ void store_at(int idx, float v) { sq[idx] = fmaf(v, v, sq[idx]); }
};

__global__ __launch_bounds__(NTHREADS, 2) void diag_conv_kernel(
    const float* g, const float* x, int n, int cout, int c, int H, int Wd, int kh, int kw, int sh,
    int sw, int ph, int pw, int dh, int dw, int OH, int OW, int samples_per_split, int splits,
    float alpha, float* out, float* ws) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int ckk = c * kh * kw;
  const int L = OH * OW;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int split = blockIdx.z;
  const int b0 = split * samples_per_split;
  const int b1 = min(n, b0 + samples_per_split);
  EpiSquares epi;
#pragma unroll
  for (int i = 0; i < 64; ++i) epi.sq[i] = 0.f;
  const ConvA Q0{x, c, H, Wd, kh, kw, sh, sw, ph, pw, dh, dw, OH, OW, ckk, 0};
  for (int b = b0; b < b1; ++b) {
    DenseMK P{g + (size_t)b * cout * L, L, cout};
    const ConvA Q(Q0, x + (size_t)b * c * H * Wd);
    gemm_tile(P, Q, m0, n0, 0, L, false, epi, smem);
  }
  float* dst = splits == 1 ? out : ws + (size_t)split * cout * ckk;
  const float scale = splits == 1 ? alpha : 1.f;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int bb = 0; bb < 2; ++bb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        int row, col;
        acc_coords<2, 2>(m0, n0, a, bb, i, row, col);
        if (row < cout && col < ckk)
          dst[(size_t)row * ckk + col] = scale * epi.sq[(a * 2 + bb) * 16 + i];
      }
}

__global__ __launch_bounds__(256) void sum_splits_kernel(const float* ws, int splits, long numel,
                                                         float alpha, float* out) {
  const long stride = (long)gridDim.x * 256;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < numel; i += stride) {
    float s = 0.f;
    for (int sp = 0; sp < splits; ++sp) s += ws[(size_t)sp * numel + i];
    out[i] = alpha * s;
  }
}

static int conv_splits(int n, int cout, int ckk) {
  const int tiles = cdiv(cout, BM) * cdiv(ckk, BN);
  int splits = 768 / tiles;
  if (splits < 1) splits = 1;
  if (splits > n) splits = n;
  const int per = cdiv(n, splits);
  return cdiv(n, per);
}

}  // namespace kfac

using namespace kfac;

extern "C" {

int kfac_diag_cov_linear(const float* g, const float* a, int n, int fout, int fin, int add_bias,
                         float alpha, float* W, float* bvec, void* stream) {
  if (!g || !a || !W || n <= 0 || fout <= 0 || fin <= 0 || (add_bias && !bvec)) return KFAC_ERR_ARG;
  if ((int64_t)n * fout * 4 > MAX_OPERAND_BYTES || (int64_t)n * fin * 4 > MAX_OPERAND_BYTES)
    return KFAC_ERR_ARG;
  const int N = fin + (add_bias ? 1 : 0);
  KFAC_LAUNCH_TILE2(diag_linear_kernel, dim3(cdiv(N, BN), cdiv(fout, BM)), (hipStream_t)stream, g,
                    a, n, fout, fin, add_bias, alpha, W, bvec);
  return launch_status();
}

size_t kfac_diag_cov_conv2d_workspace_bytes(int n, int cout, int c, int kh, int kw) {
  if (n <= 0 || cout <= 0 || c <= 0 || kh <= 0 || kw <= 0) return 0;
  const int splits = conv_splits(n, cout, c * kh * kw);
  return splits > 1 ? (size_t)splits * cout * c * kh * kw * sizeof(float) : 0;
}

int kfac_diag_cov_conv2d(const float* g, const float* x, int n, int cout, int c, int H, int W,
                         int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw,
                         float alpha, float* out, void* workspace, size_t workspace_bytes,
                         void* stream) {
  if (!g || !x || !out || n <= 0 || cout <= 0 || c <= 0 || H <= 0 || W <= 0 || kh <= 0 ||
      kw <= 0 || sh <= 0 || sw <= 0 || ph < 0 || pw < 0 || dh <= 0 || dw <= 0)
    return KFAC_ERR_ARG;
  if (H >= 16384 || W >= 16384 || kh * dh >= 16384 || kw * dw >= 16384) return KFAC_ERR_ARG;
  const int OH = (H + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
  const int OW = (W + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
  if (OH <= 0 || OW <= 0) return KFAC_ERR_ARG;
  // one sample of either tensor must fit the 30-bit operand offsets
  if ((int64_t)cout * OH * OW * 4 > MAX_OPERAND_BYTES || (int64_t)c * H * W * 4 > MAX_OPERAND_BYTES)
    return KFAC_ERR_ARG;
  const int ckk = c * kh * kw;
  const int splits = conv_splits(n, cout, ckk);
  const int per = cdiv(n, splits);
  if (splits > 1) {
    const size_t need = (size_t)splits * cout * ckk * sizeof(float);
    if (!workspace || workspace_bytes < need) return KFAC_ERR_WORKSPACE;
  }
  KFAC_LAUNCH_TILE2(diag_conv_kernel, dim3(cdiv(ckk, BN), cdiv(cout, BM), splits),
                    (hipStream_t)stream, g, x, n, cout, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, OH,
                    OW, per, splits, alpha, out, (float*)workspace);
  if (splits > 1) {
    const long numel = (long)cout * ckk;
    long blocks = (numel + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(sum_splits_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, (const float*)workspace, splits, numel, alpha, out);
  }
  return launch_status();
}

}  // extern "C"
