// Operand and epilogue functors for the tile engine in gemm_core.h.
#pragma once
#include "gemm_core.h"

namespace kfac {

// ---------------------------------------------------------------------------
// Operand functor contract used by the staging code of the tile engine.
// Elements are read with raw buffer loads (buffer_load_dword ... offen): the
// functor supplies a buffer resource over its tensor and a 32-bit BYTE offset
// per element, and an element outside the operand gets an offset beyond the
// buffer, for which the hardware returns 0 without touching memory.  So there
// is no branch, no 64-bit address arithmetic and no masking of loaded values.
//   rsrc()                    buffer resource (uniform) over [p, p + 1 GiB); valid
//                             offsets lie inside the tensor by construction
//   MS mstate(m), KS kstate(k, valid)   per-index precomputation
//   unsigned off(ms, ks)      byte offset; >= num_records when outside
//   bool is_one(ms)           the element is the constant 1 (bias augmentation)
// Offsets of valid elements are below 2^30 (tensors are limited to 1 GiB per
// call; the entry points split larger ones); an invalid row adds 2^31 and an
// invalid k adds 2^30, so every sum with an invalid part lands in [2^30, 2^32).
// ---------------------------------------------------------------------------

// The offset of a reduction index that lies outside the k range.  The arithmetic before it
// runs for every lane and the result is SELECTED: left to itself the compiler branches
// around a division for the lanes outside the range, and a write to the execution mask
// inside the reduction loop stalls the matrix pipeline (a product of two different operands
// of this kind ran at 103 instead of 127 TFLOP/s with the branches; a symmetric product,
// whose two operands share one offset, gains 1 %).
__device__ __forceinline__ unsigned k_offset_or_invalid(unsigned off, bool valid) {
  asm volatile("" : "+v"(off));      // (keeps the select from being turned back into a branch)
  return valid ? off : INV_K;
}

// Dense row-major matrix read as P(k, m) = p[k*ld + m]  (m contiguous), K rows.
// Optional last column (index M-1) that is not in memory:
//   extra == 1 : the constant 1 (bias augmentation of a Linear input)
//   extra == 2 : taken from vec[k] (bias gradient appended to a weight gradient);
//                read through a second resource and added (one of the two loads
//                of an element is always out of range, i.e. 0)
struct DenseKM {
  static constexpr int layout = KM;
  static constexpr bool has_second = true;
  static constexpr bool vec4 = true;
  // (the columns in memory; the optional last one is not)
  __device__ __forceinline__ int vec_cols() const { return extra ? M - 1 : M; }
  const float* p;
  const float* vec;
  int ld, M, extra;
  struct MS { unsigned off; unsigned off2; bool one; };
  struct KS { unsigned off; unsigned off2; };
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
    return make_rsrc(p);
  }
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc2() const {
    return make_rsrc(extra == 2 ? vec : p);
  }
  __device__ __forceinline__ bool second() const { return extra == 2; }
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    s.off = INV_M; s.off2 = INV_M; s.one = false;
    if (m < M) {
      if (extra == 1 && m == M - 1) s.one = true;
      else if (extra == 2 && m == M - 1) s.off2 = 0;
      else s.off = (unsigned)m * 4u;
    }
    return s;
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    return KS{valid ? (unsigned)(k * ld) * 4u : INV_K, valid ? (unsigned)k * 4u : INV_K};
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const { return m.off + k.off; }
  __device__ __forceinline__ unsigned off2(const MS& m, const KS& k) const { return m.off2 + k.off2; }
  __device__ __forceinline__ bool is_one(const MS& m) const { return extra == 1 && m.one; }
};

// Dense row-major matrix read as P(k, m) = p[m*ld + k]  (k contiguous), M rows.
struct DenseMK {
  static constexpr int layout = MK;
  static constexpr bool has_second = false;
  const float* p;
  int ld, M;
  struct MS { unsigned off; };
  struct KS { unsigned off; };
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
    return make_rsrc(p);
  }
  __device__ __forceinline__ MS mstate(int m) const {
    return MS{m < M ? (unsigned)(m * ld) * 4u : INV_M};
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    return KS{valid ? (unsigned)k * 4u : INV_K};
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const { return m.off + k.off; }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

// Output gradient of a Conv2d, g[n][c][hw], read as P(k=(n,pos), m=c).
struct ConvG {
  static constexpr int layout = MK;
  static constexpr bool has_second = false;
  const float* p;
  int C, HW;
  FastDiv by_hw;
  ConvG() = default;
  __host__ __device__ ConvG(const float* p_, int C_, int HW_)
      : p(p_), C(C_), HW(HW_), by_hw((unsigned)HW_) {}
  struct MS { unsigned off; };
  struct KS { unsigned off; };
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
    return make_rsrc(p);
  }
  __device__ __forceinline__ MS mstate(int m) const {
    return MS{m < C ? (unsigned)(m * HW) * 4u : INV_M};
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    const int n = by_hw.div(k);
    return KS{k_offset_or_invalid((unsigned)(n * C * HW + (k - n * HW)) * 4u, valid)};
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const { return m.off + k.off; }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

// Implicit im2col of a Conv2d input x[n][c][H][W]:
//   P(k=(n,oh,ow), m=(c,kh,kw)) = x[n][c][oh*sh - ph + kh*dh][ow*sw - pw + kw*dw]
// (0 in the padding), plus an optional trailing row of ones (m == M-1).
struct ConvA {
  static constexpr int layout = MK;
  static constexpr bool has_second = false;
  const float* p;
  int C, H, W, KH, KW, SH, SW, PH, PW, DH, DW, OH, OW, M, ones;
  FastDiv by_l, by_ow;        // divisions by OH*OW and by OW
  ConvA() = default;
  __host__ __device__ ConvA(const float* p_, int C_, int H_, int W_, int KH_, int KW_, int SH_,
                            int SW_, int PH_, int PW_, int DH_, int DW_, int OH_, int OW_, int M_,
                            int ones_)
      : p(p_), C(C_), H(H_), W(W_), KH(KH_), KW(KW_), SH(SH_), SW(SW_), PH(PH_), PW(PW_), DH(DH_),
        DW(DW_), OH(OH_), OW(OW_), M(M_), ones(ones_), by_l((unsigned)(OH_ * OW_)),
        by_ow((unsigned)OW_) {}
  __host__ __device__ ConvA(const ConvA& o, const float* p_) : ConvA(o) { p = p_; }
  // Per row m: the byte offset of (c, kh, kw) and the two patch displacements
  // packed as (dy << 16) | (dx & 0xffff), so that the 8 row states of a thread
  // take 16 registers.  dy = -32768 marks a row outside the operand (every bounds
  // test then fails; image sizes are below 16384); dx = -32768 on top of that
  // marks the row of ones.  An invalid k gets y0 = -2^20, failing the same test.
  struct MS { int off; int dydx; };
  struct KS { int off; int y0; int x0; };
  static __device__ __forceinline__ int pack(int dy, int dx) { return (dy << 16) | (dx & 0xffff); }
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
    return make_rsrc(p);
  }
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
    s.off = (c * H * W + dy * W + dx) * 4;
    return s;
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    const int n = by_l.div(k);
    const int rem = k - n * OH * OW;
    const int oh = by_ow.div(rem);
    const int ow = rem - oh * OW;
    KS s;
    s.y0 = valid ? oh * SH - PH : -(1 << 20);
    s.x0 = ow * SW - PW;
    s.off = (n * C * H * W + s.y0 * W + s.x0) * 4;
    return s;
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const {
    const int y = k.y0 + (m.dydx >> 16);
    const int x = k.x0 + (int)(short)(m.dydx & 0xffff);
    const bool ok = (unsigned)y < (unsigned)H && (unsigned)x < (unsigned)W;
    return ok ? (unsigned)(k.off + m.off) : INV_M;
  }
  __device__ __forceinline__ bool is_one(const MS& m) const {
    return ones && m.dydx == pack(-32768, -32768);
  }
};

// Implicit im2col of a Conv2d input through a copy that needs no bounds test and reads
// consecutive addresses along the reduction: the zero-padded input x~, one plane per row
// phase of the stride and per kernel column,
//   xp[n][c][ry][kw][ys][ow] = x~[n][c][ys*sh + ry][ow*sw + kw*dw],   Hs x OW each,
// with Hs = OH + (KH-1)*dh/sh, so that
//   P(k=(n,oh,ow), m=(c,kh,kw)) = xp[n][c][kh*dh % sh][kw][oh + kh*dh/sh][ow]
// is one offset per m plus one per k, and the (oh, ow) of one image are consecutive
// addresses.  (Reading x~ itself, the 16 consecutive k of a lane group fall into two or
// three pieces of rows, and the texture addresser needs 11 cycles per load instead of 4.)
// The row of ones of a layer with a bias is in memory too, OH*OW ones behind the planes of
// every image: a constant substituted after the load costs the inner loop about 7 %.
struct ConvP {
  static constexpr int layout = MK;
  static constexpr bool has_second = false;
  const float* p;
  int C, KH, KW, SH, DH, Hs, OHW, OW, M, ones;
  int image;           // floats per image: C*SH*KW planes (+ OH*OW ones)
  FastDiv by_l;        // division by OH*OW
  ConvP() = default;
  __host__ __device__ ConvP(const float* p_, int C_, int KH_, int KW_, int SH_, int DH_, int Hs_,
                            int OH_, int OW_, int M_, int ones_)
      : p(p_), C(C_), KH(KH_), KW(KW_), SH(SH_), DH(DH_), Hs(Hs_), OHW(OH_ * OW_), OW(OW_), M(M_),
        ones(ones_), image(C_ * SH_ * KW_ * Hs_ * OW_ + (ones_ ? OH_ * OW_ : 0)),
        by_l((unsigned)(OH_ * OW_)) {}
  struct MS { unsigned off; };
  struct KS { unsigned off; };
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const { return make_rsrc(p); }
  __device__ __forceinline__ MS mstate(int m) const {
    MS s;
    s.off = INV_M;
    if (m >= M) return s;
    if (ones && m == M - 1) { s.off = (unsigned)(C * SH * KW * Hs * OW) * 4u; return s; }
    const int c = m / (KH * KW);
    const int rem = m - c * KH * KW;
    const int kh = rem / KW;
    const int kw = rem - kh * KW;
    const int qy = kh * DH / SH, ry = kh * DH - qy * SH;
    s.off = (unsigned)((((c * SH + ry) * KW + kw) * Hs + qy) * OW) * 4u;
    return s;
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    const int n = by_l.div(k);
    return KS{k_offset_or_invalid((unsigned)(n * image + (k - n * OHW)) * 4u, valid)};
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const { return m.off + k.off; }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

// ---------------------------------------------------------------------------
// Epilogues
// ---------------------------------------------------------------------------

// C[row][col] = alpha*acc + beta*Cin[row][col] ; optionally also the mirrored
// element.  Cin == nullptr: the old values of C itself.
struct EpiStore {
  static constexpr bool reads_output = true;
  float* C;
  int ld, M, N;
  float alpha, beta;
  bool mirror;
  const float* Cin = nullptr;
  __device__ __forceinline__ bool reads() const { return beta != 0.f; }
  __device__ __forceinline__ float fetch(int row, int col) const {
    return (row < M && col < N) ? (Cin ? Cin : C)[(size_t)row * ld + col] : 0.f;
  }
  __device__ __forceinline__ void store_with(int row, int col, float v, float old) const {
    if (row < M && col < N) {
      const float o = alpha * v + beta * old;
      C[(size_t)row * ld + col] = o;
      if (mirror && row != col) C[(size_t)col * ld + row] = o;
    }
  }
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < M && col < N) {
      const size_t idx = (size_t)row * ld + col;
      float o = alpha * v;
      if (beta != 0.f) o += beta * (Cin ? Cin : C)[idx];
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
