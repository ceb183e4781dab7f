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
// Operand functor contract used by the staging code of the tile engine:
//   MS mstate(m), KS kstate(k)      per-index precomputation
//   const float* addr(ms, ks, ok)   ALWAYS a readable address; ok = false when the
//                                   element lies outside the operand (value -> 0)
//   bool is_one(ms)                 the element is the constant 1 (bias augmentation)
// Nothing here branches, and the value is only looked at when the chunk is
// written to LDS, so the global loads of the next chunk stay in flight while
// the MFMAs of the current one run.

// Dense row-major matrix read as P(k, m) = p[k*ld + m]  (m contiguous).
// Optional last column (index M-1) that is not in memory:
//   extra == 1 : the constant 1 (bias augmentation of a Linear input)
//   extra == 2 : taken from vec[k] (bias gradient appended to a weight gradient)
struct DenseKM {
  static constexpr int layout = KM;
  const float* p;
  const float* vec;
  int ld, M, extra;
  struct MS { const float* base; int stride; bool valid; bool one; };
  struct KS { int k; };
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    s.base = p; s.stride = 0; s.valid = false; s.one = false;
    if (m < M) {
      if (extra == 1 && m == M - 1) { s.one = true; }
      else if (extra == 2 && m == M - 1) { s.base = vec; s.stride = 1; s.valid = true; }
      else { s.base = p + m; s.stride = ld; s.valid = true; }
    }
    return s;
  }
  __device__ __forceinline__ KS kstate(int k) const { return KS{k}; }
  __device__ __forceinline__ const float* addr(const MS& m, const KS& k, bool& ok) const {
    ok = m.valid;
    return m.base + (unsigned)(k.k * m.stride);
  }
  __device__ __forceinline__ bool is_one(const MS& m) const { return extra == 1 && m.one; }
};

// Dense row-major matrix read as P(k, m) = p[m*ld + k]  (k contiguous).
struct DenseMK {
  static constexpr int layout = MK;
  const float* p;
  int ld, M;
  struct MS { const float* row; bool valid; };
  struct KS { int k; };
  __device__ __forceinline__ MS mstate(int m) const {
    return MS{m < M ? p + (size_t)m * ld : p, m < M};
  }
  __device__ __forceinline__ KS kstate(int k) const { return KS{k}; }
  __device__ __forceinline__ const float* addr(const MS& m, const KS& k, bool& ok) const {
    ok = m.valid;
    return m.row + (m.valid ? (unsigned)k.k : 0u);
  }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

// Output gradient of a Conv2d, g[n][c][hw], read as P(k=(n,pos), m=c).
struct ConvG {
  static constexpr int layout = MK;
  const float* p;
  int C, HW;
  struct MS { const float* chan; bool valid; };
  struct KS { unsigned off; };
  __device__ __forceinline__ MS mstate(int m) const {
    return MS{m < C ? p + (size_t)m * HW : p, m < C};
  }
  __device__ __forceinline__ KS kstate(int k) const {
    const int n = k / HW;
    return KS{(unsigned)(n * C * HW + (k - n * HW))};
  }
  __device__ __forceinline__ const float* addr(const MS& m, const KS& k, bool& ok) const {
    ok = m.valid;
    return m.chan + (m.valid ? k.off : 0u);
  }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

// Implicit im2col of a Conv2d input x[n][c][H][W]:
//   P(k=(n,oh,ow), m=(c,kh,kw)) = x[n][c][oh*sh - ph + kh*dh][ow*sw - pw + kw*dw]
// (0 in the padding), plus an optional trailing row of ones (m == M-1).
struct ConvA {
  static constexpr int layout = MK;
  const float* p;
  int C, H, W, KH, KW, SH, SW, PH, PW, DH, DW, OH, OW, M, ones;
  // Per row m: the element offset of (c, kh, kw) and the two patch displacements
  // packed as (dy << 16) | (dx & 0xffff) to keep the 16 row states of a thread in
  // 32 registers.  dy = -32768 marks a row outside the operand (every bounds test
  // then fails, image sizes are below 32768); dx = -32768 on top of that marks
  // the row of ones.
  struct MS { int off; int dydx; };
  struct KS { int off; int y0; int x0; };
  static __device__ __forceinline__ int pack(int dy, int dx) { return (dy << 16) | (dx & 0xffff); }
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    if (m >= M) { s.off = 0; s.dydx = pack(-32768, 0); return s; }
    if (ones && m == M - 1) { s.off = 0; s.dydx = pack(-32768, -32768); return s; }
    const int c = m / (KH * KW);
    const int rem = m - c * KH * KW;
    const int kh = rem / KW;
    const int kw = rem - kh * KW;
    const int dy = kh * DH, dx = kw * DW;
    s.dydx = pack(dy, dx);
    s.off = c * H * W + dy * W + dx;
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
  __device__ __forceinline__ const float* addr(const MS& m, const KS& k, bool& ok) const {
    const int y = k.y0 + (m.dydx >> 16);
    const int x = k.x0 + (int)(short)(m.dydx & 0xffff);
    ok = (unsigned)y < (unsigned)H && (unsigned)x < (unsigned)W;
    return p + (ok ? (unsigned)(k.off + m.off) : 0u);
  }
  __device__ __forceinline__ bool is_one(const MS& m) const {
    return ones && m.dydx == pack(-32768, -32768);
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
