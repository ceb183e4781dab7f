// Operand and epilogue functors for the tile engine in gemm_core.h.
#pragma once
#include "gemm_core.h"

namespace kfac {

// ---------------------------------------------------------------------------
// Dense row-major matrix read as P(k, m) = p[k*ld + m]  (m contiguous).
// Optional last column (index M-1) that is not in memory:
//   extra == 1 : the constant 1 (bias augmentation of a Linear input)
//   extra == 2 : taken from vec[k] (bias gradient appended to a weight gradient)
// ---------------------------------------------------------------------------
struct DenseKM {
  static constexpr int layout = KM;
  const float* p;
  const float* vec;
  int ld, M, extra;
  struct MS { int off; int kind; };   // kind: 0 outside, 1 memory, 2 ones, 3 vec
  struct KS { int off; int k; };
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    s.off = m;
    if (m >= M) s.kind = 0;
    else if (extra && m == M - 1) s.kind = extra + 1;
    else s.kind = 1;
    return s;
  }
  __device__ __forceinline__ KS kstate(int k) const { return KS{k * ld, k}; }
  __device__ __forceinline__ float load(const MS& m, const KS& k) const {
    if (m.kind == 1) return p[k.off + m.off];
    if (m.kind == 2) return 1.f;
    if (m.kind == 3) return vec[k.k];
    return 0.f;
  }
};

// Dense row-major matrix read as P(k, m) = p[m*ld + k]  (k contiguous).
struct DenseMK {
  static constexpr int layout = MK;
  const float* p;
  int ld, M;
  struct MS { int off; };             // -1 outside
  struct KS { int off; };
  __device__ __forceinline__ MS mstate(int m) const { return MS{m < M ? m * ld : -1}; }
  __device__ __forceinline__ KS kstate(int k) const { return KS{k}; }
  __device__ __forceinline__ float load(const MS& m, const KS& k) const {
    return m.off >= 0 ? p[m.off + k.off] : 0.f;
  }
};

// Output gradient of a Conv2d, g[n][c][hw], read as P(k=(n,pos), m=c).
struct ConvG {
  static constexpr int layout = MK;
  const float* p;
  int C, HW;
  struct MS { int off; };
  struct KS { int off; };
  __device__ __forceinline__ MS mstate(int m) const { return MS{m < C ? m * HW : -1}; }
  __device__ __forceinline__ KS kstate(int k) const {
    const int n = k / HW;
    return KS{n * C * HW + (k - n * HW)};
  }
  __device__ __forceinline__ float load(const MS& m, const KS& k) const {
    return m.off >= 0 ? p[m.off + k.off] : 0.f;
  }
};

// Implicit im2col of a Conv2d input x[n][c][H][W]:
//   P(k=(n,oh,ow), m=(c,kh,kw)) = x[n][c][oh*sh - ph + kh*dh][ow*sw - pw + kw*dw]
// (0 in the padding), plus an optional trailing row of ones (m == M-1).
struct ConvA {
  static constexpr int layout = MK;
  const float* p;
  int C, H, W, KH, KW, SH, SW, PH, PW, DH, DW, OH, OW, M, ones;
  struct MS { int off; int dy; int dx; };   // dy == -2^30: outside; dy == -2^29: ones row
  struct KS { int off; int y0; int x0; };
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    if (m >= M) { s.off = 0; s.dy = -(1 << 30); s.dx = 0; return s; }
    if (ones && m == M - 1) { s.off = 0; s.dy = -(1 << 29); s.dx = 0; return s; }
    const int c = m / (KH * KW);
    const int rem = m - c * KH * KW;
    const int kh = rem / KW;
    const int kw = rem - kh * KW;
    s.dy = kh * DH;
    s.dx = kw * DW;
    s.off = c * H * W + s.dy * W + s.dx;
    return s;
  }
  __device__ __forceinline__ KS kstate(int k) const {
    const int n = k / (OH * OW);
    const int rem = k - n * OH * OW;
    const int oh = rem / OW;
    const int ow = rem - oh * OW;
    KS s;
    s.y0 = oh * SH - PH;
    s.x0 = ow * SW - PW;
    s.off = n * C * H * W + s.y0 * W + s.x0;
    return s;
  }
  __device__ __forceinline__ float load(const MS& m, const KS& k) const {
    if (m.dy == -(1 << 30)) return 0.f;
    if (m.dy == -(1 << 29)) return 1.f;
    const int y = k.y0 + m.dy;
    const int x = k.x0 + m.dx;
    if ((unsigned)y < (unsigned)H && (unsigned)x < (unsigned)W) return p[k.off + m.off];
    return 0.f;
  }
};

// ---------------------------------------------------------------------------
// Epilogues
// ---------------------------------------------------------------------------

// C[row][col] = alpha*acc + beta*C_old ; optionally also the mirrored element.
struct EpiStore {
  float* C;
  int ld, M, N;
  float alpha, beta;
  bool mirror;
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < M && col < N) {
      const size_t idx = (size_t)row * ld + col;
      float o = alpha * v;
      if (beta != 0.f) o += beta * C[idx];
      C[idx] = o;
      if (mirror && row != col) C[(size_t)col * ld + row] = o;
    }
  }
};

// raw partial sums of one k-split into a tile-packed workspace
struct EpiPartial {
  float* ws;      // already offset to this (split, tile)
  int m0, n0, M, N, tn;   // tn = tile width
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < M && col < N) ws[(row - m0) * tn + (col - n0)] = v;
  }
};

}  // namespace kfac
