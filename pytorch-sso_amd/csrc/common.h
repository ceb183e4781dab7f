// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/kfac_hip.h"

namespace kfac {

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// Dynamic LDS sizes are registered once per kernel (required above 64 KiB, as
// for the 148 KiB of the diagonal-block kernel; harmless below).
bool enable_large_lds(const void* kernel, int bytes);

#define KFAC_LAUNCH_TILE2(kernel, grid, stream, ...)                                         \
  do {                                                                                       \
    constexpr int lds_bytes_ = kfac::Cfg<2, 2>::SMEM_FLOATS * (int)sizeof(float);            \
    if (kfac::enable_large_lds((const void*)(kernel), lds_bytes_))                           \
      hipLaunchKernelGGL((kernel), (grid), dim3(kfac::NTHREADS), lds_bytes_, (stream),       \
                         __VA_ARGS__);                                                       \
  } while (0)

// A factor of a stride-1, bias-free Conv2d by spatial correlations
// (factor_conv_taps.hip).  conv_a_taps returns -1 when the geometry is not
// covered; the caller then uses the im2col kernel.
bool conv_a_taps_applicable(int c, int kh, int kw, int sh, int sw, int add_bias);
size_t conv_a_taps_workspace(int n, int c, int H, int W, int kh, int kw, int ph, int pw, int dh,
                             int dw);
double conv_a_taps_executed_flops(int n, int c, int H, int W, int kh, int kw, int ph, int pw,
                                  int dh, int dw);   // 0 when the geometry is not covered
int conv_a_taps(const float* x, int n, int c, int H, int W, int kh, int kw, int ph, int pw, int dh,
                int dw, float alpha, float beta, const float* A_prev, float* A, void* workspace,
                size_t workspace_bytes, hipStream_t stream);

// Copies a small host table to device memory at `dev` (4-byte aligned, `bytes` rounded up to
// a multiple of 4 are written) as kernel arguments of a few tiny launches on `stream`: no
// hipMemcpy, so the caller stays capturable and never waits for the device.  The host
// memory may be reused as soon as this returns.
void upload_table(const void* host, size_t bytes, void* dev, hipStream_t stream);

// The stride-1 k x k input factors of several layers at once (factor_conv_taps.hip): every
// geometry must be one that conv_a_taps covers (conv_a_taps_workspace(...) > 0).
struct TapsJob {
  const float* x;
  int n, c, H, W, kh, kw, ph, pw, dh, dw;
  float alpha, beta;
  const float* A_prev;
  float* A;
};
size_t conv_a_taps_grouped_workspace(int count, const TapsJob* jobs);
double conv_a_taps_grouped_executed_flops(int count, const TapsJob* jobs);
int conv_a_taps_grouped(int count, const TapsJob* jobs, void* workspace, size_t workspace_bytes,
                        hipStream_t stream);

// Blocks per piece of the cut reductions of a launch of 128x128 tiles (0: none is cut).
// `work` = sum over the tiles of their reduction length in blocks, `longest` = the longest
// of them: with the work spread evenly over the chip's resident workgroups (3 per CU) the
// launch would last work / 768 block times, and it cannot end before its longest tile does
// (which shares its compute unit with two other workgroups until the launch thins out).
// Where the longest tile is the longer of the two, reductions are cut into pieces that are
// work items of the same launch and store raw partial tiles; a short launch afterwards adds
// the pieces of every cut tile up in order (splitk_sum).
constexpr int MIN_PIECE_BLOCKS = 4;
inline int piece_blocks(long work, int longest) {
  const long even = work / 768 + 1;
  if (longest <= MIN_PIECE_BLOCKS || 3 * (long)longest <= 4 * even) return 0;
  const long pb = even / 2 > MIN_PIECE_BLOCKS ? even / 2 : MIN_PIECE_BLOCKS;
  return pb >= longest ? 0 : (int)pb;
}

// Tiles' worth of MFMA work in the T(T+1)/2 upper tiles of a symmetric product with T tiles
// per side: a diagonal tile leaves out its 32x32 blocks below the diagonal, 6 of 16 for a
// 128-wide tile of four waves, 1 of 4 for a 64-wide tile of one.
inline double syrk_tile_units(int T, int w) {
  const double diag = w == 2 ? 10. / 16. : 3. / 4.;
  return (double)T * (T - 1) / 2 + T * diag;
}

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? KFAC_OK : KFAC_ERR_LAUNCH;
}

}  // namespace kfac
