// Reduction of k-split partial tiles of a symmetric product, shared by the single-product
// and the grouped factor builders.  Partials are tile-packed: [split][tile][TS x TS].
#pragma once
#include "operands.h"

namespace kfac {

// Sum the k-split partials of one tile in a fixed order and apply the epilogue
// (+ mirror).  One workgroup (256 threads) owns 64 consecutive elements of a tile row
// (seg_idx = row inside the tile * TS/64 + segment):
// 16 float4 groups x 16 split lanes; lane s adds splits s, s+16, ... and the 16
// lane sums are then added in lane order, so the result does not depend on
// scheduling.
template <int TS>
__device__ __forceinline__ void syrk_reduce_many(const float* ws, int d, int T, int ntiles,
                                                 int splits, float* C, const float* Cin,
                                                 float alpha, float beta, int tile, int seg_idx) {
  __shared__ float4 red[16][16];
  int bi, bj;
  upper_tile(tile, T, bi, bj);
  constexpr int SEGS = TS / 64;
  const int lrow = seg_idx / SEGS;
  const int seg = seg_idx - lrow * SEGS;
  const int row = bi * TS + lrow;
  const int col0 = bj * TS + seg * 64;
  if (row >= d || col0 >= d) return;
  const int g = threadIdx.x & 15;
  const int sl = threadIdx.x >> 4;
  const size_t e = (size_t)lrow * TS + seg * 64 + 4 * g;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  const size_t stride = (size_t)ntiles * (TS * TS);
  const float* base = ws + (size_t)tile * (TS * TS) + e;
#pragma unroll 4
  for (int sp = sl; sp < splits; sp += 16) {
    const float4 v = *reinterpret_cast<const float4*>(base + (size_t)sp * stride);
    acc.x += v.x;
    acc.y += v.y;
    acc.z += v.z;
    acc.w += v.w;
  }
  red[sl][g] = acc;
  __syncthreads();
  if (sl == 0) {
    float4 s = red[0][g];
#pragma unroll
    for (int k = 1; k < 16; ++k) {
      const float4 v = red[k][g];
      s.x += v.x;
      s.y += v.y;
      s.z += v.z;
      s.w += v.w;
    }
    const float vals[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int col = col0 + 4 * g + k;
      if (col < d) {
        const size_t idx = (size_t)row * d + col;
        float o = alpha * vals[k];
        if (beta != 0.f) o += beta * (Cin ? Cin : C)[idx];
        C[idx] = o;
        if (bi != bj) C[(size_t)col * d + row] = o;
      }
    }
  }
}

// The same reduction for few splits and many tiles: one workgroup owns 32 rows x 64
// columns of a tile, a thread two float4 groups, and walks the splits with four
// loads in flight.  The mirrored block goes through LDS, so that it is written in
// runs of 32 elements as well.
template <int TS>
__device__ __forceinline__ void syrk_reduce_tile(const float* ws, int d, int T, int ntiles,
                                                 int splits, float* C, const float* Cin,
                                                 float alpha, float beta, int tile, int rblk,
                                                 int cblk) {
  __shared__ float mir[32][65];
  int bi, bj;
  upper_tile(tile, T, bi, bj);
  const int r0 = rblk * 32, c0 = cblk * 64;      // inside the tile
  if (bi * TS + r0 >= d || bj * TS + c0 >= d) return;
  const int g = threadIdx.x & 15, rr = threadIdx.x >> 4;
  const size_t stride = (size_t)ntiles * (TS * TS);
  const float* base = ws + (size_t)tile * (TS * TS) + (size_t)(r0 + rr) * TS + c0 + 4 * g;
  float4 acc[2] = {make_float4(0.f, 0.f, 0.f, 0.f), make_float4(0.f, 0.f, 0.f, 0.f)};
#pragma unroll 2
  for (int sp = 0; sp < splits; ++sp) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float4 v = *reinterpret_cast<const float4*>(base + (size_t)sp * stride + h * 16 * TS);
      acc[h].x += v.x;
      acc[h].y += v.y;
      acc[h].z += v.z;
      acc[h].w += v.w;
    }
  }
  const float* prev = Cin ? Cin : C;
  float o[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float vals[4] = {acc[h].x, acc[h].y, acc[h].z, acc[h].w};
    const int row = bi * TS + r0 + rr + 16 * h;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int col = bj * TS + c0 + 4 * g + k;
      const bool in = row < d && col < d;
      o[h][k] = alpha * vals[k] + ((beta != 0.f && in) ? beta * prev[(size_t)row * d + col] : 0.f);
    }
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = bi * TS + r0 + rr + 16 * h;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int col = bj * TS + c0 + 4 * g + k;
      if (row < d && col < d) C[(size_t)row * d + col] = o[h][k];
      mir[rr + 16 * h][4 * g + k] = o[h][k];
    }
  }
  if (bi == bj) return;
  __syncthreads();
  // element (c, r) of the mirrored block: 8 of its rows per pass, 32 elements each
  const int mr = threadIdx.x & 31;
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int mc = (threadIdx.x >> 5) + 8 * pass;
    const int row = bi * TS + r0 + mr, col = bj * TS + c0 + mc;
    if (row < d && col < d) C[(size_t)col * d + row] = mir[mr][mc];
  }
}

}  // namespace kfac
