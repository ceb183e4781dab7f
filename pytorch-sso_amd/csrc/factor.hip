// Kronecker factor builders: symmetric products  C = alpha * P^T P + beta * C
// over the upper-triangular 128x128 tiles of C, mirrored in the epilogue.
#include "common.h"
#include "operands.h"
#include "syrk_reduce.h"

#include <string.h>

#include <atomic>

namespace kfac {

// Which kernels already had their dynamic-LDS limit raised, per device.  A fixed table
// of atomics: trivially destructible, so nothing of this library runs at process exit
// (objects with destructors in a shared library are torn down in an order that other
// libraries' exit handlers do not expect).
bool enable_large_lds(const void* kernel, int bytes) {
  constexpr int MAX_DEVICES = 64, CAP = 96;
  static std::atomic<const void*> done[MAX_DEVICES][CAP];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  if (dev >= 0 && dev < MAX_DEVICES) {
    for (int i = 0; i < CAP; ++i) {
      const void* k = done[dev][i].load(std::memory_order_acquire);
      if (k == kernel) return true;
      if (k != nullptr) continue;
      if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) !=
          hipSuccess)
        return false;
      // publish in the first free slot from here on (two threads setting the attribute
      // of one kernel at the same time both succeed; a duplicate entry is harmless)
      for (; i < CAP; ++i) {
        const void* expected = nullptr;
        if (done[dev][i].compare_exchange_strong(expected, kernel, std::memory_order_acq_rel) ||
            expected == kernel)
          break;
      }
      return true;
    }
  }
  // table full or device index out of its range: set the attribute on every call
  return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) ==
         hipSuccess;
}

constexpr int UPLOAD_WORDS = 960;     // 3840 bytes of the 4 KiB a launch may carry as arguments
struct UploadChunk {
  unsigned w[UPLOAD_WORDS];
};
__global__ __launch_bounds__(256) void upload_kernel(UploadChunk chunk, unsigned* dst, int words) {
  for (int i = threadIdx.x; i < words; i += 256) dst[i] = chunk.w[i];
}

void upload_table(const void* host, size_t bytes, void* dev, hipStream_t stream) {
  const size_t words = (bytes + 3) / 4;
  for (size_t w0 = 0; w0 < words; w0 += UPLOAD_WORDS) {
    UploadChunk c;
    const size_t n = words - w0 < (size_t)UPLOAD_WORDS ? words - w0 : (size_t)UPLOAD_WORDS;
    const size_t nb = (w0 + n) * 4 <= bytes ? n * 4 : bytes - w0 * 4;
    c.w[n - 1] = 0;
    memcpy(c.w, (const char*)host + w0 * 4, nb);
    hipLaunchKernelGGL(upload_kernel, dim3(1), dim3(256), 0, stream, c, (unsigned*)dev + w0,
                       (int)n);
  }
}

// Tile configuration and k-split of a symmetric d x d product reduced over K:
// 64-wide single-wave tiles for small factors (a 128-wide tile would be mostly
// padding), 128-wide tiles otherwise; enough k-splits to put about 8 waves on
// every SIMD, each split at least 128 deep.
struct SyrkPlan {
  int w;        // waves per tile side: 1 -> 64x64 tiles, 2 -> 128x128
  int ts;       // tile size
  int T;        // tiles per side
  int ntiles;   // upper-triangular tiles
  int splits;
  int cps;      // chunks (of the configuration's KC) per split
};

static SyrkPlan plan_syrk(int d, long K) {
  SyrkPlan p;
  p.w = d <= 256 ? 1 : 2;
  p.ts = 64 * p.w;
  p.T = cdiv(d, p.ts);
  p.ntiles = p.T * (p.T + 1) / 2;
  const int kc = p.w == 1 ? Cfg<1, 1>::KC : Cfg<2, 2>::KC;
  const long nchunks = (K + kc - 1) / kc;
  const long target = 2048 / (p.w * p.w);
  long splits = target / p.ntiles;
  if (splits < 1) splits = 1;
  const long min_chunks = 128 / kc;      // each split at least 128 deep
  const long max_splits = nchunks / min_chunks > 0 ? nchunks / min_chunks : 1;
  if (splits > max_splits) splits = max_splits;
  long cps = (nchunks + splits - 1) / splits;
  if (cps < 1) cps = 1;
  splits = (nchunks + cps - 1) / cps;
  if (splits < 1) splits = 1;
  if (p.w == 2) {
    // All workgroups of up to 3 per CU are resident at once and share the CU's matrix
    // cores, so the launch takes (workgroups on the fullest CU) x (chunks per split):
    // a few more splits can take a whole round off.  Every extra split costs one more
    // partial tile written and read (the last term, in chunk times).
    const int ncu = 256;
    auto cost = [&](long s, long c) {
      return (double)cdiv((int)(s * p.ntiles), ncu) * (c + 3) + (s > 1 ? 0.035 * s * p.ntiles : 0.);
    };
    double best = cost(splits, cps);
    long best_s = splits, best_cps = cps;
    for (long s = splits + 1; s <= max_splits && s * p.ntiles <= 3 * ncu; ++s) {
      const long c = (nchunks + s - 1) / s;
      if ((nchunks + c - 1) / c != s) continue;
      if (cost(s, c) < best) {
        best = cost(s, c);
        best_s = s;
        best_cps = c;
      }
    }
    splits = best_s;
    cps = best_cps;
  }
  p.splits = (int)splits;
  p.cps = (int)cps;
  return p;
}

template <class OP, int W>
__global__ __launch_bounds__(64 * W * W, W == 2 ? 3 : 1) void syrk_kernel(OP op, int d, int K, int T, int ntiles,
                                                          int splits, int chunks_per_split,
                                                          float* C, const float* Cin,
                                                          float alpha, float beta, float* ws) {
  constexpr int TS = 64 * W;
  constexpr int KC = Cfg<W, W>::KC;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // work item = (split, tile), tile fastest: the tiles of one split read the
  // same rows of the input, so they are kept on one XCD
  const int item = xcd_remap(blockIdx.y * ntiles + blockIdx.x, ntiles * splits);
  const int tile = item % ntiles;
  const int split = item / ntiles;
  int bi, bj;
  upper_tile(tile, T, bi, bj);
  const int kbeg = split * chunks_per_split * KC;
  int kend = kbeg + chunks_per_split * KC;
  if (kend > K) kend = K;
  if (splits == 1) {
    EpiStore epi{C, d, d, d, alpha, beta, bi != bj, Cin};
    gemm_tile_cfg<W, W, true>(op, op, bi * TS, bj * TS, kbeg, kend, bi == bj, epi, smem);
  } else {
    EpiPartial epi{ws + ((size_t)split * ntiles + tile) * (TS * TS), bi * TS, bj * TS, d, d, TS};
    gemm_tile_cfg<W, W, true>(op, op, bi * TS, bj * TS, kbeg, kend, bi == bj, epi, smem);
  }
}

template <int TS>
__global__ __launch_bounds__(256) void syrk_reduce_kernel(const float* ws, int d, int T,
                                                           int ntiles, int splits, float* C,
                                                           const float* Cin, float alpha,
                                                           float beta) {
  syrk_reduce_many<TS>(ws, d, T, ntiles, splits, C, Cin, alpha, beta, blockIdx.x, blockIdx.y);
}

template <int TS>
__global__ __launch_bounds__(256) void syrk_reduce_tile_kernel(const float* ws, int d, int T,
                                                                int ntiles, int splits, float* C,
                                                                const float* Cin, float alpha,
                                                                float beta) {
  syrk_reduce_tile<TS>(ws, d, T, ntiles, splits, C, Cin, alpha, beta, blockIdx.x, blockIdx.y,
                       blockIdx.z);
}

template <class OP, int W>
static void launch_syrk_cfg(const OP& op, const SyrkPlan& p, int d, int64_t K, float alpha,
                            float beta, const float* Cin, float* C, void* workspace,
                            hipStream_t stream) {
  constexpr int TS = 64 * W;
  constexpr int lds_bytes = Cfg<W, W>::SMEM_FLOATS * (int)sizeof(float);
  if (!enable_large_lds((const void*)syrk_kernel<OP, W>, lds_bytes)) return;
  hipLaunchKernelGGL((syrk_kernel<OP, W>), dim3(p.ntiles, p.splits), dim3(64 * W * W), lds_bytes,
                     stream, op, d, (int)K, p.T, p.ntiles, p.splits, p.cps, C, Cin, alpha, beta,
                     (float*)workspace);
  if (p.splits > 16) {
    hipLaunchKernelGGL((syrk_reduce_kernel<TS>), dim3(p.ntiles, TS * (TS / 64)), dim3(256), 0,
                       stream, (const float*)workspace, d, p.T, p.ntiles, p.splits, C, Cin, alpha,
                       beta);
  } else if (p.splits > 1) {
    hipLaunchKernelGGL((syrk_reduce_tile_kernel<TS>), dim3(p.ntiles, TS / 32, TS / 64), dim3(256),
                       0, stream, (const float*)workspace, d, p.T, p.ntiles, p.splits, C, Cin,
                       alpha, beta);
  }
}

template <class OP>
static int launch_syrk(const OP& op, int d, int64_t K, float alpha, float beta, const float* Cin,
                       float* C, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  const SyrkPlan p = plan_syrk(d, (long)K);
  if (p.splits > 1) {
    const size_t need = (size_t)p.splits * p.ntiles * p.ts * p.ts * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) return KFAC_ERR_WORKSPACE;
  }
  if (p.w == 1)
    launch_syrk_cfg<OP, 1>(op, p, d, K, alpha, beta, Cin, C, workspace, stream);
  else
    launch_syrk_cfg<OP, 2>(op, p, d, K, alpha, beta, Cin, C, workspace, stream);
  return launch_status();
}

}  // namespace kfac

using namespace kfac;

extern "C" {

int kfac_abi_version(void) { return 2; }

size_t kfac_factor_workspace_bytes(int d, int64_t K) {
  if (d <= 0 || K <= 0) return 0;
  const SyrkPlan p = plan_syrk(d, (long)K);
  return p.splits > 1 ? (size_t)p.splits * p.ntiles * p.ts * p.ts * sizeof(float) : 0;
}

// Operand offsets are 30-bit byte offsets: an input larger than 1 GiB is consumed
// in slices along its leading dimension, each slice accumulating into C.
static int64_t slice_len(int64_t total, int64_t elems_per_unit) {
  const int64_t max_units = (MAX_OPERAND_BYTES / 4) / elems_per_unit;
  return max_units < 1 ? 0 : (total < max_units ? total : max_units);
}

// MFMA flops one launch_syrk executes: every (tile, split) workgroup runs whole chunks of
// KC reduction steps on a full ts x ts tile (padding and the k tail included); a diagonal
// tile leaves out its 32x32 blocks below the diagonal.
static double syrk_executed_flops(int d, int64_t K) {
  const SyrkPlan p = plan_syrk(d, (long)K);
  const int kc = p.w == 1 ? Cfg<1, 1>::KC : Cfg<2, 2>::KC;
  const double chunks = (double)((K + kc - 1) / kc);
  return syrk_tile_units(p.T, p.w) * chunks * kc * 2.0 * p.ts * p.ts;
}

double kfac_factor_executed_flops(int d, int64_t K) {
  if (d <= 0 || K <= 0) return 0.;
  return syrk_executed_flops(d, K);
}

double kfac_factor_conv_a_executed_flops(int n, int c, int H, int W, int kh, int kw, int sh,
                                         int sw, int ph, int pw, int dh, int dw, int add_bias) {
  if (n <= 0 || c <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 ||
      ph < 0 || pw < 0 || dh <= 0 || dw <= 0)
    return 0.;
  const int OH = (H + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
  const int OW = (W + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
  if (OH <= 0 || OW <= 0) return 0.;
  const int64_t image = (int64_t)c * H * W;
  const int64_t step = slice_len(n, image);
  if (step == 0) return 0.;
  const int d = c * kh * kw + (add_bias ? 1 : 0);
  double total = 0.;
  for (int64_t n0 = 0; n0 < n; n0 += step) {
    const int cnt = (int)(n - n0 < step ? n - n0 : step);
    if (kh == 1 && kw == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && !add_bias) {
      total += syrk_executed_flops(d, (int64_t)cnt * H * W);
      continue;
    }
    if (conv_a_taps_applicable(c, kh, kw, sh, sw, add_bias)) {
      const double t = conv_a_taps_executed_flops(cnt, c, H, W, kh, kw, ph, pw, dh, dw);
      if (t > 0.) {
        total += t;
        continue;
      }
    }
    total += syrk_executed_flops(d, (int64_t)cnt * OH * OW);
  }
  return total;
}

size_t kfac_factor_conv_a_workspace_bytes(int n, int c, int H, int W, int kh, int kw, int sh,
                                          int sw, int ph, int pw, int dh, int dw, int add_bias) {
  if (n <= 0 || c <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 ||
      ph < 0 || pw < 0 || dh <= 0 || dw <= 0)
    return 0;
  const int OH = (H + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
  const int OW = (W + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
  if (OH <= 0 || OW <= 0) return 0;
  const int64_t image = (int64_t)c * H * W;
  const int64_t step = slice_len(n, image);
  if (step == 0) return 0;
  const int d = c * kh * kw + (add_bias ? 1 : 0);
  size_t need = kfac_factor_workspace_bytes(d, step * OH * OW);
  if (conv_a_taps_applicable(c, kh, kw, sh, sw, add_bias)) {
    const size_t t = conv_a_taps_workspace((int)step, c, H, W, kh, kw, ph, pw, dh, dw);
    if (t > need) need = t;
    if (n % step) {
      const size_t t2 = conv_a_taps_workspace((int)(n % step), c, H, W, kh, kw, ph, pw, dh, dw);
      if (t2 > need) need = t2;
    }
  }
  return need;
}

int kfac_factor_linear(const float* x, int64_t rows, int f, int64_t ldx, int add_bias,
                       float alpha, float beta, const float* C_prev, float* C, void* workspace,
                       size_t workspace_bytes, void* stream) {
  if (!x || !C || rows <= 0 || f <= 0 || ldx < f) return KFAC_ERR_ARG;
  const int d = f + (add_bias ? 1 : 0);
  if ((int64_t)d * d * 4 > MAX_OPERAND_BYTES) return KFAC_ERR_ARG;
  const int64_t step = slice_len(rows, ldx);
  if (step == 0) return KFAC_ERR_ARG;
  for (int64_t r0 = 0; r0 < rows; r0 += step) {
    const int64_t cnt = rows - r0 < step ? rows - r0 : step;
    DenseKM op{x + r0 * ldx, nullptr, (int)ldx, d, add_bias ? 1 : 0};
    const int st = launch_syrk(op, d, cnt, alpha, r0 == 0 ? beta : 1.f,
                               r0 == 0 ? C_prev : nullptr, C, workspace, workspace_bytes,
                               (hipStream_t)stream);
    if (st != KFAC_OK) return st;
  }
  return KFAC_OK;
}

int kfac_factor_conv_a(const float* x, int n, int c, int H, int W, int kh, int kw, int sh, int sw,
                       int ph, int pw, int dh, int dw, int add_bias, float alpha, float beta,
                       const float* C_prev, float* C, void* workspace, size_t workspace_bytes,
                       void* stream) {
  if (!x || !C || n <= 0 || c <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 ||
      sw <= 0 || ph < 0 || pw < 0 || dh <= 0 || dw <= 0)
    return KFAC_ERR_ARG;
  if (H >= 16384 || W >= 16384 || kh * dh >= 16384 || kw * dw >= 16384) return KFAC_ERR_ARG;
  const int OH = (H + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
  const int OW = (W + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
  if (OH <= 0 || OW <= 0) return KFAC_ERR_ARG;
  const int64_t dd = (int64_t)c * kh * kw + (add_bias ? 1 : 0);
  if (dd * dd * 4 > MAX_OPERAND_BYTES) return KFAC_ERR_ARG;
  const int d = (int)dd;
  const int64_t image = (int64_t)c * H * W;
  const int64_t step = slice_len(n, image);   // (offsets into the padding are never used)
  if (step == 0) return KFAC_ERR_ARG;
  for (int64_t n0 = 0; n0 < n; n0 += step) {
    const int cnt = (int)(n - n0 < step ? n - n0 : step);
    const float bslice = n0 == 0 ? beta : 1.f;
    const float* prev = n0 == 0 ? C_prev : nullptr;
    if (kh == 1 && kw == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && !add_bias) {
      // a pointwise convolution: M is the input itself, viewed as [c, n*H*W]
      ConvG op{x + n0 * image, c, H * W};
      const int st = launch_syrk(op, d, (int64_t)cnt * H * W, alpha, bslice, prev, C, workspace,
                                 workspace_bytes, (hipStream_t)stream);
      if (st != KFAC_OK) return st;
      continue;
    }
    if (conv_a_taps_applicable(c, kh, kw, sh, sw, add_bias)) {
      const int st = conv_a_taps(x + n0 * image, cnt, c, H, W, kh, kw, ph, pw, dh, dw, alpha,
                                 bslice, prev, C, workspace, workspace_bytes, (hipStream_t)stream);
      if (st == KFAC_OK) continue;
      if (st != -1) return st;
    }
    ConvA op{x + n0 * image, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, OH, OW, d, add_bias ? 1 : 0};
    const int st = launch_syrk(op, d, (int64_t)cnt * OH * OW, alpha, bslice, prev, C, workspace,
                               workspace_bytes, (hipStream_t)stream);
    if (st != KFAC_OK) return st;
  }
  return KFAC_OK;
}

int kfac_factor_conv_g(const float* g, int n, int c, int h, int w, float alpha, float beta,
                       const float* C_prev, float* C, void* workspace, size_t workspace_bytes,
                       void* stream) {
  if (!g || !C || n <= 0 || c <= 0 || h <= 0 || w <= 0) return KFAC_ERR_ARG;
  if ((int64_t)c * c * 4 > MAX_OPERAND_BYTES) return KFAC_ERR_ARG;
  const int64_t image = (int64_t)c * h * w;
  const int64_t step = slice_len(n, image);
  if (step == 0) return KFAC_ERR_ARG;
  for (int64_t n0 = 0; n0 < n; n0 += step) {
    const int cnt = (int)(n - n0 < step ? n - n0 : step);
    ConvG op{g + n0 * image, c, h * w};
    const int st = launch_syrk(op, c, (int64_t)cnt * h * w, alpha, n0 == 0 ? beta : 1.f,
                               n0 == 0 ? C_prev : nullptr, C, workspace, workspace_bytes,
                               (hipStream_t)stream);
    if (st != KFAC_OK) return st;
  }
  return KFAC_OK;
}

}  // extern "C"
