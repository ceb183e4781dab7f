// Batched damped SPD inverse:  dst_i = (src_i + damp_i * I)^-1  for a whole set
// of matrices of different sizes in one sequence of launches.
//
//   1. copy the upper triangle of src into dst and add damp to the diagonal
//      (damp is either given, or computed on the device from the traces of a
//      pair of Kronecker factors: the pi-damping split);
//   2. blocked right-looking Cholesky  S = U^T U  (upper, in place in dst) with
//      128-wide panels: one workgroup factors AND inverts the 128x128 diagonal
//      block in LDS; the row panel is a product with that small inverse; the
//      trailing update is a symmetric rank-128 product on the MFMA tile engine.
//      Panels are grouped: the rows of the current group receive each panel's
//      update in the launch that factors the next diagonal block (that block's
//      workgroup applies it to its own tile first, tile workgroups to the rest,
//      so that the chip is not idle while the latency-bound block is factored:
//      two launches per panel), the rows beyond the group receive the whole group
//      in one deeper product;
//   3. Y = U^-1 by recursive doubling over the 128-blocks:
//      Y12 = -Y11 * U12 * Y22, two MFMA products per level, log2(n/128) levels;
//   4. dst = Y Y^T on the MFMA tile engine (upper tiles, mirrored).
//
// Every launch covers all matrices that still have work at that step (matrices
// are processed in descending size order so the active ones form a prefix),
// so small factors ride along with the large ones instead of getting a launch
// sequence each.
#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

#include "common.h"
#include "operands.h"

namespace kfac {

struct MatDesc {
  const float* src;
  float* U;      // Cholesky factor, then the inverse: dst (the workspace slot when only Y is wanted)
  float* Y;      // inverse of the Cholesky factor, n*n: the workspace slot, or the caller's
                 // buffer when Y itself is the result
  int n;
  int T;         // number of 128-blocks
  float damp;    // given damping, or sqrt(damping) in pi mode
  int partner;   // -1: damp is final; else index of the other factor of the pair
  int is_a;      // pi mode: 1 -> damp*pi, 0 -> damp/pi
  int out;       // position in the caller's info array
  float trace;
  int rev;       // 1: the work matrix is src with rows and columns reversed (see run_batched)
  float* W;      // rev only: receives the upper Cholesky factor of the inverse, else nullptr
  int noinv;     // 1: the explicit inverse is not wanted, Y is the result (Y Y^T = inverse)
  int pad;
};

constexpr int SETUP_CHUNK = 48;
struct DescChunk {
  MatDesc d[SETUP_CHUNK];
};

__global__ void inv_setup_kernel(DescChunk chunk, MatDesc* table, int offset, int count) {
  const int i = threadIdx.x;
  if (i < count) table[offset + i] = chunk.d[i];
}

// trace of src (one workgroup per matrix)
__global__ __launch_bounds__(256) void inv_trace_kernel(MatDesc* table) {
  __shared__ float red[256];
  MatDesc& m = table[blockIdx.x];
  const int n = m.n;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) s += m.src[(size_t)i * n + i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) m.trace = red[0];
}

__device__ __forceinline__ float effective_damp(const MatDesc* table, const MatDesc& m) {
  if (m.partner < 0) return m.damp;
  const MatDesc& o = table[m.partner];
  const float ta = m.is_a ? m.trace / m.n : o.trace / o.n;
  const float tg = m.is_a ? o.trace / o.n : m.trace / m.n;
  const float pi = sqrtf(ta / tg);
  return m.is_a ? m.damp * pi : m.damp / pi;
}

// U = upper tiles of (src + damp I); also clears info
__global__ __launch_bounds__(256) void inv_copy_damp_kernel(const MatDesc* table, int* info,
                                                            const WorkList wl) {
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  if (local == 0 && threadIdx.x == 0) info[m.out] = 0;
  int bi, bj;
  upper_tile(local, m.T, bi, bj);
  const float damp = effective_damp(table, m);
  const int n = m.n;
  // 8 loads in flight per thread, then 8 stores
  for (int e0 = threadIdx.x; e0 < BM * BN; e0 += 256 * 8) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int e = e0 + 256 * k;
      const int row = bi * BM + (e >> 7);
      const int col = bj * BN + (e & 127);
      const size_t at = m.rev ? (size_t)(n - 1 - row) * n + (n - 1 - col) : (size_t)row * n + col;
      v[k] = (row < n && col < n) ? m.src[at] : 0.f;
      if (row == col) v[k] += damp;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int e = e0 + 256 * k;
      const int row = bi * BM + (e >> 7);
      const int col = bj * BN + (e & 127);
      if (row < n && col < n) m.U[(size_t)row * n + col] = v[k];
    }
  }
}

// ---------------------------------------------------------------------------
// 128x128 diagonal block: Cholesky (upper) and its inverse, in LDS.
// ---------------------------------------------------------------------------
constexpr int DB = 128;          // diagonal block size
constexpr int DLD = DB + 1;      // LDS leading dimension
constexpr int DIAG_SMEM_BYTES = 2 * DB * DLD * (int)sizeof(float);

__device__ __forceinline__ float lane_value(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src_lane));
}

// One wave: acc(32x32) = sum_{k<K} A(k, i) * B(k, j) with operands in LDS,
//   A(k, i) = a[k*a_ks + i*a_is],  B(k, j) = b[k*b_ks + j*b_js]   (K a multiple of 32).
// Result element t of lane (r, h): row 8*(t/4) + 4h + t%4, column r.
__device__ __forceinline__ v16f lds_mma32(const lds_f* a, int a_ks, int a_is, const lds_f* b,
                                          int b_ks, int b_js, int K) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  v16f acc;
#pragma unroll
  for (int t = 0; t < 16; ++t) acc[t] = 0.f;
  const lds_f* pa = a + h * a_ks + r * a_is;
  const lds_f* pb = b + h * b_ks + r * b_js;
  // 32 deep at a time: the 32 operand reads of a slice are issued together, and those of the
  // next slice before the 16 MFMAs of this one
  float av[16], bv[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    av[i] = pa[2 * i * a_ks];
    bv[i] = pb[2 * i * b_ks];
  }
  for (int k0 = 0; k0 < K; k0 += 32) {
    float an[16], bn[16];
    if (k0 + 32 < K) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        an[i] = pa[(k0 + 32 + 2 * i) * a_ks];
        bn[i] = pb[(k0 + 32 + 2 * i) * b_ks];
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[i], acc, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      av[i] = an[i];
      bv[i] = bn[i];
    }
  }
  return acc;
}

// The elimination of a 32-row strip, two rows per step, on 32x32 blocks that live in the
// accumulator registers of v_mfma_f32_32x32x2_f32: element t of lane (r = lane & 31,
// h = lane >> 5) is (row 8*(t/4) + 4*h + t%4, column r), so row c of a block is ONE register
// (index 4*(c/8) + c%4) in the 32 lanes of half (c/4)%2, lane = column, and rows c, c+1
// (c even) are neighbouring registers in the same half.
//   L: the diagonal leaf, a full symmetric 32x32 block (Schur complement of the rows above);
//   P: the same rows of another 32 columns (a block of the row panel, or of [ . | identity]).
// A step finishes rows c and c+1:  with the 2x2 pivot block [p00 p01; p01 p11] of L,
//   w0 = L[c] / sqrt(p00),  u01 = p01 / sqrt(p00),  w1 = (L[c+1] - u01 w0) / sqrt(p11 - u01^2)
// are rows c, c+1 of U (the same combination y0, y1 of P's rows: those rows of the second
// block), and the rows below get  X[i][j] -= w0[i] y0[j] + w1[i] y1[j]  as ONE rank-2 matrix
// instruction per block: its reduction slot 0 is the lanes 0-31 of the operand registers,
// slot 1 the lanes 32-63, so (w0 | w1) in the two halves of one register is the B operand
// (lane = column j) and, negated and zeroed in the lanes i <= c+1, the A operand (lane = row
// i; by the symmetry of L its rows are its columns).  Both rows live in one half, so one
// v_permlane32_swap moves the second into the other half; apart from that and the three
// pivot entries (v_readlane) no value changes lanes.  The chain from step to step is
//   matrix instruction -> pivots -> two 1/sqrt -> w1 -> swap -> matrix instruction.
// The finished rows go to LDS as they are made, straight from the operand registers
// (`leaf_rows`: where U_qq goes, or a block of LDS that nothing reads for a wave that only
// needs the multipliers; `blk_rows`: the second block's rows).  Below its diagonal U_qq is
// left with rounding noise there; whoever copies it out writes zeros instead.
// `pmin`, `piv`: the smallest pivot so far and all 32 of them, for the caller's check.
// With P = rows of the panel the strip ends as U[q][*] = U_qq^-T A[q][*] without a
// triangular solve; with P = [pending | identity] as the rows of U^-T.
template <int H>
__device__ __forceinline__ float pair_operand(float x0, float x1) {
  // both valid in the lanes of half H -> x0 in lanes 0-31, x1 in lanes 32-63
  // (the instruction swaps lanes 32-63 of its first register with lanes 0-31 of its second)
  const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x0),
                                                   __builtin_bit_cast(unsigned, x1), false, false);
  return __builtin_bit_cast(float, H ? sw[1] : sw[0]);
}

template <int C>
__device__ __forceinline__ void elim_pair(v16f& L, v16f& P, lds_f* leaf_rows, lds_f* blk_rows,
                                          int r, float& pmin, float (&piv)[32]) {
  constexpr int T = 4 * (C >> 3) + (C & 3), H = (C >> 2) & 1;
  const float v0 = L[T], v1 = L[T + 1];
  const float p00 = lane_value(v0, 32 * H + C);
  const float p01 = lane_value(v0, 32 * H + C + 1);
  const float p11 = lane_value(v1, 32 * H + C + 1);
  const float r0 = __builtin_amdgcn_rsqf(p00);
  const float u01 = p01 * r0;
  const float d = fmaf(-u01, u01, p11);
  const float r1 = __builtin_amdgcn_rsqf(d);
  const float w0 = v0 * r0;
  const float w1 = fmaf(-u01, w0, v1) * r1;
  const float xb = pair_operand<H>(w0, w1);
  const float xa = r > C + 1 ? -xb : 0.f;
  if (C < 30) L = __builtin_amdgcn_mfma_f32_32x32x2f32(xa, xb, L, 0, 0, 0);
  // (nothing below moves in front of that instruction: the second block's work belongs in
  // the wait for its result)
  __builtin_amdgcn_sched_barrier(0);
  const float y0 = P[T] * r0;
  const float y1 = fmaf(-u01, y0, P[T + 1]) * r1;
  const float pb = pair_operand<H>(y0, y1);
  if (C < 30) P = __builtin_amdgcn_mfma_f32_32x32x2f32(xa, pb, P, 0, 0, 0);
  // the finished rows: the operand registers hold row C in the lanes 0-31 and row C+1 in the
  // lanes 32-63, so one store writes both (the pointers carry the lane's row and column)
  leaf_rows[C * DLD] = xb;
  blk_rows[C * DLD] = pb;
  pmin = fminf(fminf(pmin, p00), d);
  piv[C] = p00;
  piv[C + 1] = d;
  __builtin_amdgcn_sched_barrier(0);
}

template <int C>
__device__ __forceinline__ void elim_from(v16f& L, v16f& P, lds_f* leaf_rows, lds_f* blk_rows,
                                          int r, float& pmin, float (&piv)[32]) {
  if constexpr (C < 32) {
    elim_pair<C>(L, P, leaf_rows, blk_rows, r, pmin, piv);
    elim_from<C + 2>(L, P, leaf_rows, blk_rows, r, pmin, piv);
  }
}

// Factors and inverts diagonal block p of matrix m: one workgroup of DIAG_THREADS threads
// (12 waves) with DIAG_SMEM_BYTES of LDS at dsm: S, the block (upper triangle and the whole
// diagonal 32-blocks; finished rows of U replace it strip by strip), and Z, the rows of
// U_pp^-T.
// Four strips of 32 rows.  In strip q each of the waves 0-3 holds the leaf (its own copy:
// the multipliers of a step come from it) and ONE further block of the same rows: a block
// of the row panel to the right of the leaf (3 - q of them), or a block of the same rows of
// Z (q + 1 of them, the last one starting as the identity).  That is four blocks in every
// strip, one per wave, and the inverse Y_pp = Z^T is complete when the last strip is: no back
// substitution, no doubling.  The updates by finished strips happen in LDS, by the other
// waves: strip q-1's update of the rows of strip q first (four blocks, waves 4-7: this is
// on the chain), its update of the rows further down while strip q is eliminated (at most
// five blocks, waves 4-11); those waves also write the finished rows of strip q-1 to global
// memory meanwhile, so that only the last strip's are left at the end.
constexpr int DIAG_THREADS = 768;

// `pending`: the row panel above (block row p-1) has not been applied to this block yet
// (the launch that holds this workgroup applies it to the rest of block row p meanwhile).
__device__ __forceinline__ void diag_block(const MatDesc& m, int p, int* info, float* dsm,
                                           bool pending) {
  lds_f* const S = (lds_f*)dsm;
  lds_f* const Z = S + DB * DLD;
  const int n = m.n;
  const int r0 = p * DB;
  const int nb = min(DB, n - r0);
  const int t = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);     // (provably uniform: scalar branches)
  const int lane = t & 63;
  const int r = lane & 31, h = lane >> 5;
  // the waves that eliminate the strips go first wherever they share a SIMD with the others
  if (wave < 4) __builtin_amdgcn_s_setprio(3);

  // load the upper triangle; pad with the identity up to 128.  All loads of a thread are
  // issued before the first is used: one memory round trip for the block.
  // (raw buffer loads: no 64-bit address per element, and the elements outside the
  // triangle cost no memory access)
  {
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(m.U + (size_t)r0 * n + r0);
    // (pending: tile (p-1, p) of U, all of its 128 rows, in the same round trip)
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(m.U + ((size_t)r0 - DB) * n + r0);
    constexpr int PER = (DB * DB + DIAG_THREADS - 1) / DIAG_THREADS;
    float v[PER], a[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = u * DIAG_THREADS + t;
      const int i = e >> 7, j = e & 127;
      // (the diagonal 32-blocks in full, their lower triangles from the upper one: a strip
      // reads its leaf as a plain symmetric block)
      const bool in = i < nb && j < nb && (j >= i || (j >> 5) == (i >> 5));
      v[u] = buffer_load(rs, in ? (unsigned)(min(i, j) * n + max(i, j)) * 4u : INV_M);
      if (pending) a[u] = buffer_load(ra, (i < DB && j < nb) ? (unsigned)(i * n + j) * 4u : INV_M);
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = u * DIAG_THREADS + t;
      if (e >= DB * DB) break;
      const int i = e >> 7, j = e & 127;
      const bool in = i < nb && j < nb && (j >= i || (j >> 5) == (i >> 5));
      const bool pad = (i >= nb || j >= nb) && i == j;
      S[i * DLD + j] = in ? v[u] : (pad ? 1.f : 0.f);
      if (pending) Z[i * DLD + j] = a[u];
    }
  }
  __syncthreads();
  // S -= W^T W, W = tile (p-1, p) of U (in Z for now), 128 deep, by 32x32 blocks: the four
  // blocks of the first strip's rows now (waves 4-7, one per SIMD), the other six while
  // that strip is eliminated (it writes Z in the columns of its own block only, which
  // those six do not read; later strips find W spent)
  auto pending_block = [&](int blk) {
    int bi, bj;
    upper_tile(blk, 4, bi, bj);
    const v16f acc = lds_mma32(Z + 32 * bi, DLD, 1, Z + 32 * bj, DLD, 1, DB);
    lds_f* const c = S + (32 * bi + 4 * h) * DLD + 32 * bj + r;
    float old[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) old[e] = c[(8 * (e >> 2) + (e & 3)) * DLD];
#pragma unroll
    for (int e = 0; e < 16; ++e) c[(8 * (e >> 2) + (e & 3)) * DLD] = old[e] - acc[e];
  };
  if (pending && wave >= 4 && wave < 8) pending_block(wave - 4);
  // (the loop over the strips starts with a barrier)

  typedef __attribute__((address_space(1))) float global_f;
  global_f* const gU = (global_f*)(m.U + (size_t)r0 * n + r0);
  global_f* const gY = (global_f*)(m.Y + (size_t)r0 * n + r0);
  // rows [32 qs, 32 qs + 32) of U and the same columns of Y = Z^T, by `nthr` threads
  auto write_strip = [&](int qs, int tid, int nthr) {
    for (int e0 = 0; e0 < 32 * DB; e0 += 8 * nthr) {
      float u[8], y[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int e = min(e0 + k * nthr + tid, 32 * DB - 1);
        const int iu = 32 * qs + (e >> 7), ju = e & 127;      // U[iu][ju]
        const int iy = e >> 5, jy = 32 * qs + (e & 31);       // Y[iy][jy] = Z[jy][iy]
        u[k] = iu <= ju ? S[iu * DLD + ju] : 0.f;
        y[k] = iy <= jy ? Z[jy * DLD + iy] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int e = e0 + k * nthr + tid;
        if (e >= 32 * DB) break;
        const int iu = 32 * qs + (e >> 7), ju = e & 127;
        const int iy = e >> 5, jy = 32 * qs + (e & 31);
        if (iu < nb && ju < nb) gU[iu * n + ju] = u[k];
        if (iy < nb && jy < nb) gY[iy * n + jy] = y[k];
      }
    }
  };

  const int nq = (nb + 31) / 32;
  // Strip qs's update of block row i, by `nw` of the waves from 4 on, block by block in LDS
  // (item k of the row goes to wave 4 + (first + k) % nw):
  //   S(i, j) -= U[qs][i]^T U[qs][j]  (i <= j),     Z(i, s) -= U[qs][i]^T Z[qs][s]  (s <= qs)
  auto update_row = [&](int qs, int i, int first, int nw) {
    const lds_f* const above = S + 32 * qs * DLD;
    const lds_f* const zabove = Z + 32 * qs * DLD;
    for (int k = 0; k < nq - i + qs + 1; ++k) {
      if ((first + k) % nw != wave - 4) continue;
      const bool in_s = k < nq - i;
      const int col = in_s ? i + k : k - (nq - i);         // block column of S, or of Z
      const v16f acc = lds_mma32(above + 32 * i, DLD, 1, (in_s ? above : zabove) + 32 * col,
                                 DLD, 1, 32);
      lds_f* const c = (in_s ? S : Z) + (32 * i + 4 * h) * DLD + 32 * col + r;
      // (a block of Z below the diagonal starts at zero: its first update, by the strip of
      // its column, finds it uninitialised)
      const bool fresh = !in_s && col == qs;
      float old[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) old[e] = fresh ? 0.f : c[(8 * (e >> 2) + (e & 3)) * DLD];
#pragma unroll
      for (int e = 0; e < 16; ++e) c[(8 * (e >> 2) + (e & 3)) * DLD] = old[e] - acc[e];
    }
    return nq - i + qs + 1;
  };
  for (int q = 0; q < nq; ++q) {
    const int c0 = 32 * q;
    const int rest = nq - q - 1;       // 32-blocks of the row panel to the right of the leaf
    const bool strip_wave = wave < 4 && wave < nq;
    const bool panel = wave < rest;    // this wave's second block: panel block jb, or block s
    const int jb = q + 1 + wave;       // of the rows of Z
    const int s = wave - rest;
    // the rows of this strip meet the update by the strip above (nq blocks, one per wave)
    if (wave >= 4 && q > 0) update_row(q - 1, q, 0, 4);
    __syncthreads();
    if (wave < 4) {
      if (strip_wave) {
        v16f L, P;
        const lds_f* const lsrc = S + (c0 + 4 * h) * DLD + c0 + r;
        const lds_f* const psrc =
            (panel ? S + c0 * DLD + 32 * jb : Z + c0 * DLD + 32 * s) + 4 * h * DLD + r;
#pragma unroll
        for (int e = 0; e < 16; ++e) L[e] = lsrc[(8 * (e >> 2) + (e & 3)) * DLD];
        if (panel || s < q) {
#pragma unroll
          for (int e = 0; e < 16; ++e) P[e] = psrc[(8 * (e >> 2) + (e & 3)) * DLD];
        } else {
#pragma unroll
          for (int e = 0; e < 16; ++e) P[e] = 8 * (e >> 2) + 4 * h + (e & 3) == r ? 1.f : 0.f;
        }
        // (block (3, 0) of S, below its diagonal, is never used; the lane's column made
        // opaque per strip, so that the lane masks derived from it are computed where they
        // are used instead of being kept, and spilled, across the loop over the strips)
        int rr = r;
        asm volatile("" : "+v"(rr));
        lds_f* const leaf_rows = (wave == 0 ? S + c0 * DLD + c0 : S + 96 * DLD) + h * DLD + r;
        lds_f* const blk_rows = (panel ? S + c0 * DLD + 32 * jb : Z + c0 * DLD + 32 * s) + h * DLD + r;
        float pmin = 1.f, piv[32];
        // every wave has its copy of the leaf in registers before wave 0 writes U_qq over it
        // (the waves 4-7 and the idle ones pass the same barrier below)
        __syncthreads();
        elim_from<0>(L, P, leaf_rows, blk_rows, rr, pmin, piv);
        // LAPACK's info: the first pivot that is not positive.  A NaN anywhere in the leaf
        // reaches a pivot and from there every later one, so the last pivot stands for them.
        if (wave == 0 && (!(pmin > 0.f) || !(piv[31] > 0.f))) {
          int bad = 0;
#pragma unroll
          for (int c = 31; c >= 0; --c)
            if (!(piv[c] > 0.f)) bad = r0 + c0 + c + 1;
          int* const out = info + m.out;
          if (lane == 0 && *out == 0) *out = bad;
        }
      } else {
        __syncthreads();
      }
    } else {
      __syncthreads();
      // meanwhile: the strip above's update of the rows further down, and its rows to memory
      if (q == 0 && pending && wave < 10) pending_block(wave);      // blocks 4..9
      if (q > 0) {
      int first = 0;
      for (int i = q + 1; i < nq; ++i) first += update_row(q - 1, i, first, 8);
      write_strip(q - 1, t - 256, DIAG_THREADS - 256);
      }
    }
    __syncthreads();
  }
  write_strip(nq - 1, t, DIAG_THREADS);
}

__global__ __launch_bounds__(DIAG_THREADS) void potrf_diag_kernel(const MatDesc* table, int p,
                                                                   int* info) {
  extern __shared__ __attribute__((aligned(16))) float dsm[];
  diag_block(table[blockIdx.x], p, info, dsm, false);
}

// row panel of the blocked Cholesky: U[p, j] = Ypp^T * A[p, j], j > p
__global__ __launch_bounds__(NTHREADS) void potrf_panel_kernel(const MatDesc* table, int p,
                                                               const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  const int bj = p + 1 + local;
  if (bj >= m.T) return;
  const int n = m.n;
  const int r0 = p * DB;
  DenseKM P{m.Y + (size_t)r0 * n + r0, nullptr, n, DB, 0};
  DenseKM Q{m.U + (size_t)r0 * n, nullptr, n, n, 0};
  EpiStore epi{m.U + (size_t)r0 * n, n, DB, n, 1.f, 0.f, false};
  gemm_tile(P, Q, 0, bj * BN, 0, DB, false, epi, smem);
}

// Tile (bi <= bj) number `local` of the trailing update of block rows [row_lo, row_hi).
__device__ __forceinline__ bool trail_tile(int T, int row_lo, int row_hi, int local, int& bi,
                                           int& bj) {
  const int hi = min(row_hi, T);
  if (row_lo >= hi) return false;
  if (row_hi >= T) {
    // all remaining rows: walk the upper triangle of the (T - row_lo)^2 block grid
    const int Tr = T - row_lo;
    if (local >= Tr * (Tr + 1) / 2) return false;
    upper_tile(xcd_remap(local, Tr * (Tr + 1) / 2), Tr, bi, bj);
    bi += row_lo;
    bj += row_lo;
    return true;
  }
  // a few rows: rectangular walk, tiles left of the diagonal exit
  const int width = T - row_lo;
  const int rr = local / width;
  bi = row_lo + rr;
  bj = row_lo + (local - rr * width);
  return bi < hi && bj >= bi;
}

// trailing update with the block rows [kb0, kb0 + nk) of U:
//   A[i, j] -= sum_k U[k, i]^T U[k, j]   for block rows row_lo <= i < row_hi, j >= i.
// The Cholesky runs in groups of GROUP_BLOCKS diagonal blocks: inside a group each step
// updates only the remaining rows of that group (nk = 1), and the rows beyond it receive
// the whole group at once (nk = GROUP_BLOCKS), which cuts the read-modify-write passes over
// the trailing matrix by that factor (a rank-128 update of a large trailing matrix is
// bound by memory traffic, not by the matrix cores).  Taller groups run no faster (measured
// up to 16: the tiles that ride along with a diagonal block are hidden either way) and
// cost accuracy: the float32 error of the inverse of a 9217^2 factor with condition number
// 9e2 grows from 2.2e-5 (height 1) over 5.2e-5 (4; scipy's float32 LU inverse: 4.7e-5) to
// 1.0e-4 (16), because a deeper product accumulates more terms before it meets the
// entry it nearly cancels.
constexpr int GROUP_BLOCKS = 4;
// The last TAIL_BLOCKS diagonal blocks of the largest matrices form one group: the deeper
// update of the rows beyond a group is a launch that lasts as long as one 512-deep tile
// (50 us) however few tiles it has, while the rank-128 updates of a short trailing matrix
// all fit beside the next diagonal block (up to three tiles per compute unit there).
// (with the tiles packed three to a workgroup: config 3 inversion 4.75 / 4.77 / 4.90 / 5.16 ms
// with 16 / 24 / 32 / 40; a 3201^2 and a 1601^2 matrix 1.68 / 1.58 / 1.53 / 1.53 ms; three
// 9217 / 4097 / 4097 matrices 10.12 / 10.03 / 9.95 / 9.92 ms and 10.58 ms with 64)
constexpr int TAIL_BLOCKS = 24;

__global__ __launch_bounds__(NTHREADS, 3) void potrf_trail_kernel(const MatDesc* table, int kb0,
                                                               int nk, int row_lo, int row_hi,
                                                               const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  int bi, bj;
  if (!trail_tile(m.T, row_lo, row_hi, local, bi, bj)) return;
  const int n = m.n;
  DenseKM P{m.U + (size_t)kb0 * DB * n, nullptr, n, n, 0};
  EpiStore epi{m.U, n, n, n, -1.f, 1.f, false};
  gemm_tile(P, P, bi * BM, bj * BN, 0, nk * DB, bi == bj, epi, smem);
}

// Diagonal blocks p and, beside them, the part of panel p-1's update that nothing needs
// before the next row panel:   A[i,j] -= U[p-1,i]^T U[p-1,j]   for block rows
// row_lo <= i < row_hi (row_lo = p + 1: row p got its update in a launch of its own).
// The first `ndiag` workgroups take one diagonal block each (potrf_diag_kernel's work),
// the others `tpw` tiles each.  The launch carries the diagonal block's LDS, so one
// workgroup runs per CU: the tile workgroups use the CUs that the few diagonal blocks
// leave idle, for about as long as a diagonal block takes; a launch with more tiles than
// CUs puts up to three tiles into a workgroup, as many waves per CU as in a launch of
// their own.
constexpr int STEP_TILES_PER_WG = DIAG_THREADS / NTHREADS;
static_assert(STEP_TILES_PER_WG * SMEM_FLOATS * (int)sizeof(float) <= DIAG_SMEM_BYTES,
              "the tiles of a workgroup share the diagonal block's LDS");

__global__ __launch_bounds__(DIAG_THREADS) void potrf_step_kernel(const MatDesc* table, int p,
                                                                   int* info, int ndiag,
                                                                   int row_lo, int row_hi, int tpw,
                                                                   const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float dsm[];
  if ((int)blockIdx.x < ndiag) {
    diag_block(table[blockIdx.x], p, info, dsm, true);
    return;
  }
  // A tile is the work of four waves.  A launch with more tiles than compute units packs
  // `tpw` (up to three) of them into a workgroup, each group of four waves with its own
  // 40 KB of the launch's LDS; every tile of this launch reduces over the same 128 rows, so
  // the groups meet at the same barriers (a group that has returned no longer counts).
  const int group = (int)threadIdx.x / NTHREADS;
  if (group >= tpw) return;
  const int item = ((int)blockIdx.x - ndiag) * tpw + group;
  if (item >= wl.cum[wl.n]) return;
  int mat, local, bi, bj;
  work_find_item(wl, item, mat, local);
  if (!trail_tile(table[mat].T, row_lo, row_hi, local, bi, bj)) return;
  if (bj == p) return;                       // tile (p, p): the diagonal block's own workgroup
  const MatDesc m = table[mat];
  const int n = m.n;
  DenseKM P{m.U + (size_t)(p - 1) * DB * n, nullptr, n, n, 0};
  EpiStore epi{m.U, n, n, n, -1.f, 1.f, false};
  gemm_tile(P, P, bi * BM, bj * BN, 0, DB, bi == bj, epi, dsm + group * SMEM_FLOATS);
}

// The row panel for launches of few tiles: the same 128x128x128 product, but by 16 waves
// with one 32x32 block each instead of 4 waves with four.  A tile is a chain of
// dependent-issue MFMAs, 256 per wave (7.8 us) in the tile engine and 64 here, and at the
// end of a factorisation nothing else runs beside it.  Both operands are fetched whole (32
// loads per thread in flight) into 128 KB of LDS.
constexpr int FINE_THREADS = 1024;
constexpr int FINE_SMEM_BYTES = 2 * DB * DB * (int)sizeof(float);
constexpr int FINE_MAX_TILES = 256;      // one workgroup per CU

__global__ __launch_bounds__(FINE_THREADS) void potrf_fine_kernel(const MatDesc* table, int p,
                                                                  const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float fsm[];
  lds_f* const tp = (lds_f*)fsm;
  lds_f* const tq = tp + DB * DB;
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  const int n = m.n;
  const int bj = p + 1 + local;
  if (bj >= m.T) return;
  // P(k, i) = Y_pp;  Q(k, j) = A[p, bj], j < qw;  C[i][j] = U[p, bj] over Q
  const float* P = m.Y + (size_t)p * DB * n + p * DB;
  const float* Q = m.U + (size_t)p * DB * n + bj * DB;
  float* C = m.U + (size_t)p * DB * n + bj * DB;
  const int qw = min(DB, n - bj * DB);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int r = lane & 31, h = lane >> 5;
  const int wr = wave >> 2, wc = wave & 3;

  const int mm = t & (DB - 1), kq = t >> 7;
  const __amdgpu_buffer_rsrc_t rp = make_rsrc(P), rq = make_rsrc(Q);
  float vp[16], vq[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const unsigned off = (unsigned)((kq + 8 * i) * n + mm) * 4u;
    vp[i] = buffer_load(rp, off);
    vq[i] = buffer_load(rq, mm < qw ? off : INV_M);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    tp[(kq + 8 * i) * DB + mm] = vp[i];
    tq[(kq + 8 * i) * DB + mm] = vq[i];
  }
  __syncthreads();
  const v16f acc = lds_mma32(tp + 32 * wr, DB, 1, tq + 32 * wc, DB, 1, DB);
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int row = 32 * wr + 8 * (e >> 2) + 4 * h + (e & 3), col = 32 * wc + r;
    if (col < qw) C[(size_t)row * n + col] = acc[e];
  }
}

// The same product for launches of very few tiles (at most SUB_MAX_TILES): every tile is
// dealt to four workgroups, so that four CUs' matrix cores work on it.  The row panel
// overwrites its own right-hand operand, so the pieces must not share columns: four
// 128x32 column strips, four 32x32 blocks each.  8 waves: a wave does one block over half
// of the 128-deep reduction and the halves are added through LDS.
constexpr int SUB_THREADS = 512;
constexpr int SUB_SMEM_BYTES = DB * (128 + 32) * (int)sizeof(float);
constexpr int SUB_MAX_TILES = 64;        // 4 workgroups per tile, one workgroup per CU

__global__ __launch_bounds__(SUB_THREADS) void potrf_sub_kernel(const MatDesc* table, int p,
                                                                const WorkList wl) {
  constexpr int WP = 128, WQ = 32;
  extern __shared__ __attribute__((aligned(16))) float fsm[];
  lds_f* const tp = (lds_f*)fsm;
  lds_f* const tq = tp + DB * WP;
  int mat, item;
  work_find(wl, mat, item);
  const int local = item >> 2, sj = item & 3;
  const MatDesc m = table[mat];
  const int n = m.n;
  const int bj = p + 1 + local;
  if (bj >= m.T) return;
  const float* P = m.Y + (size_t)p * DB * n + p * DB;
  const float* Q = m.U + (size_t)p * DB * n + bj * DB;
  float* C = m.U + (size_t)p * DB * n + bj * DB;
  const int qw = min(DB, n - bj * DB);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int r = lane & 31, h = lane >> 5;
  const int br = wave & 3, khalf = wave >> 2;
  const int row0 = 32 * br, col0 = WQ * sj;         // of this wave's block in the tile

  const __amdgpu_buffer_rsrc_t rp = make_rsrc(P), rq = make_rsrc(Q);
  float vp[WP / 4], vq[WQ / 4];
#pragma unroll
  for (int i = 0; i < WP / 4; ++i) {
    const int idx = t + SUB_THREADS * i;
    vp[i] = buffer_load(rp, (unsigned)((idx / WP) * n + idx % WP) * 4u);
  }
#pragma unroll
  for (int i = 0; i < WQ / 4; ++i) {
    const int idx = t + SUB_THREADS * i;
    const int k = idx / WQ, col = WQ * sj + idx % WQ;
    vq[i] = buffer_load(rq, col < qw ? (unsigned)(k * n + col) * 4u : INV_M);
  }
#pragma unroll
  for (int i = 0; i < WP / 4; ++i) tp[t + SUB_THREADS * i] = vp[i];
#pragma unroll
  for (int i = 0; i < WQ / 4; ++i) tq[t + SUB_THREADS * i] = vq[i];
  __syncthreads();
  const v16f acc = lds_mma32(tp + 64 * khalf * WP + 32 * br, WP, 1, tq + 64 * khalf * WQ, WQ, 1,
                             64);
  __syncthreads();
  // the second halves of the reduction travel through LDS (the operands are spent)
  lds_f* const red = tp + br * 1024;
  if (khalf == 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) red[e * 64 + lane] = acc[e];
  }
  __syncthreads();
  if (khalf == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = row0 + 8 * (e >> 2) + 4 * h + (e & 3), col = col0 + r;
      const float v = acc[e] + red[e * 64 + lane];
      if (col < qw) C[(size_t)row * n + col] = v;
    }
  }
}

// ---- Y = U^-1 by balanced recursive halving over the 128-blocks ---------------
// Depth d cuts the T blocks of a matrix into 2^d nearly equal segments
// (boundaries floor(j*T/2^d)); the merge of the two children X1, X2 of a
// depth-d segment computes  Y12 = -Y11 * U12 * Y22, one tile per pair of a block of
// X1 and a block of X2.  A launch walks the tiles of all merges of its depth.
struct MergeTile {
  int X1, b1, X2, b2, it, jt;
  bool valid;
};

struct Segment {
  int p0, mid, p1;
  __host__ __device__ int tiles() const { return (mid - p0) * (p1 - mid); }
};

__host__ __device__ inline Segment segment(int P, int depth, int T) {
  Segment s;
  s.p0 = (int)(((long)P * T) >> depth);
  s.p1 = (int)(((long)(P + 1) * T) >> depth);
  s.mid = (int)(((long)(2 * P + 1) * T) >> (depth + 1));
  return s;
}

__host__ __device__ inline int merge_tiles(int T, int depth) {
  int total = 0;
  for (int P = 0; P < (1 << depth); ++P) total += segment(P, depth, T).tiles();
  return total;
}

// Tile `local` of the merges at `depth`, longest reduction first: a launch lasts at least
// as long as its longest tile (up to T/2 blocks on ONE compute unit, shared with two other
// workgroups), so those start first and the launch ends on its one-block tiles.  The
// reduction of the first product grows with the column of the tile (`fast` = column, the
// tiles of a column share the Y22 panel), that of the second shrinks with the row (`fast`
// = row, its tiles share the Y11 panel).  The halves of all segments of a depth differ by
// at most one block, so rank r (0 = longest) holds one tile per `slow` index of every
// segment, except the last rank, which only the longer segments have.
__device__ __forceinline__ MergeTile merge_tile(const MatDesc& m, int depth, int local,
                                                bool by_column) {
  MergeTile t;
  t.valid = false;
  const int T = m.T, nseg = 1 << depth;
  int fmax = 0, s_all = 0, s_top = 0;
  for (int P = 0; P < nseg; ++P) {
    const Segment sg = segment(P, depth, T);
    const int rows = sg.mid - sg.p0, cols = sg.p1 - sg.mid;
    const int f = by_column ? rows : cols, sl = by_column ? cols : rows;
    if (f == 0 || sl == 0) continue;
    if (f > fmax) { fmax = f; s_top = 0; }
    if (f == fmax) s_top += sl;
    s_all += sl;
  }
  if (fmax == 0) return t;
  const int full = (fmax - 1) * s_all;
  if (local >= full + s_top) return t;
  int r, q;
  if (local < full) {
    r = local / s_all;
    q = local - r * s_all;
  } else {
    r = fmax - 1;
    q = local - full;
  }
  for (int P = 0; P < nseg; ++P) {
    const Segment sg = segment(P, depth, T);
    const int rows = sg.mid - sg.p0, cols = sg.p1 - sg.mid;
    const int f = by_column ? rows : cols, sl = by_column ? cols : rows;
    if (f == 0 || sl == 0 || f <= r) continue;
    if (q >= sl) { q -= sl; continue; }
    if (by_column) {
      t.it = r;
      t.jt = q;
    } else {
      t.it = q;
      t.jt = f - 1 - r;
    }
    t.X1 = sg.p0 * DB;
    t.b1 = rows * DB;
    t.X2 = sg.mid * DB;
    t.b2 = min(cols * DB, m.n - t.X2);
    t.valid = true;
    return t;
  }
  return t;
}

// first product:  W^T[j][i] = sum_{k <= j} Y22[k][j] * U12[i][k], stored at
// Y[X2 rows][X1 cols] (the unused lower triangle of Y)
__global__ __launch_bounds__(NTHREADS) void trtri_w_kernel(const MatDesc* table, int depth,
                                                           const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  const MergeTile t = merge_tile(m, depth, local, false);
  if (!t.valid) return;
  const int n = m.n;
  DenseKM P{m.Y + (size_t)t.X2 * n + t.X2, nullptr, n, t.b2, 0};
  DenseMK Q{m.U + (size_t)t.X1 * n + t.X2, n, t.b1};
  EpiStore epi{m.Y + (size_t)t.X2 * n + t.X1, n, t.b2, t.b1, 1.f, 0.f, false};
  gemm_tile(P, Q, t.jt * BM, t.it * BN, 0, min(t.b2, (t.jt + 1) * DB), false, epi, smem);
}

// second product:  Y12[i][j] = - sum_{k >= i} Y11[i][k] * W^T[j][k]
__global__ __launch_bounds__(NTHREADS) void trtri_y_kernel(const MatDesc* table, int depth,
                                                           const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  const MergeTile t = merge_tile(m, depth, local, true);
  if (!t.valid) return;
  const int n = m.n;
  DenseMK P{m.Y + (size_t)t.X1 * n + t.X1, n, t.b1};
  DenseMK Q{m.Y + (size_t)t.X2 * n + t.X1, n, t.b2};
  EpiStore epi{m.Y + (size_t)t.X1 * n + t.X2, n, t.b1, t.b2, -1.f, 0.f, false};
  gemm_tile(P, Q, t.it * BM, t.jt * BN, t.it * DB, t.b1, false, epi, smem);
}

// Which upper tile (bi <= bj) of Y Y^T a workgroup takes.  The tiles of a column bj all
// reduce over k >= bj*128 (same length) and share the operand panel Y[bj rows], and the
// work of a column, (bj + 1) * (T - bj), varies smoothly with bj.  Workgroups go to the
// 8 XCDs (one L2 each) in turn by dispatch index, so XCD x is given the columns
// bj = x, x + 8, ... (equal work within 3 %, a panel is read by one L2 only), first
// column (longest reduction) first.  The classes differ a little in tile count while every
// XCD gets the same number of workgroups: the surplus tiles of a class, which are its
// shortest, go to the workgroups that the smaller classes leave without a tile.
__device__ __forceinline__ int column_class_size(int T, int x) {
  if (x > T - 1) return 0;
  const int c = (T - 1 - x) / 8 + 1;
  return c * (x + 1) + 4 * c * (c - 1);
}

__device__ __forceinline__ void column_class_tile(int x, int t, int& bi, int& bj) {
  bj = x;
  while (t >= bj + 1) {
    t -= bj + 1;
    bj += 8;
  }
  bi = t;
}

__device__ __forceinline__ void lauum_tile(int T, int local, int& bi, int& bj) {
  const int ntiles = T * (T + 1) / 2;
  const int g = (int)blockIdx.x;
  const int x = g & 7;
  const int s8 = (g - local) & 7;                  // where the matrix starts in the grid, mod 8
  int deficit_before = 0, slots_x = 0, size_x = 0, first_x = 0;
  int slots[8], size[8];
#pragma unroll
  for (int y = 0; y < 8; ++y) {
    const int first = (y - s8 + 8) & 7;            // first workgroup of this matrix on XCD y
    slots[y] = max(0, (ntiles - first + 7) / 8);
    size[y] = column_class_size(T, y);
    if (y == x) {
      slots_x = slots[y];
      size_x = size[y];
      first_x = first;
    }
  }
  const int t = (local - first_x) / 8;
  if (t < size_x) {
    column_class_tile(x, t, bi, bj);
    return;
  }
#pragma unroll
  for (int y = 0; y < 8; ++y)
    if (y < x) deficit_before += max(0, slots[y] - size[y]);
  int r = deficit_before + (t - size_x);           // rank among the tiles without a workgroup
  (void)slots_x;
#pragma unroll
  for (int z = 0; z < 8; ++z) {
    const int excess = max(0, size[z] - slots[z]);
    if (r >= 0 && r < excess) {
      column_class_tile(z, slots[z] + r, bi, bj);
      return;
    }
    r -= excess;
  }
  bi = bj = 0;       // not reached: the classes hold exactly ntiles tiles
}

// C[f(row)][f(col)] = v and its mirror image, f(i) = base + sign * i: the identity, or the
// reversal i -> n - 1 - i that undoes the reversed read of a matrix factored back to front
struct EpiSymFlip {
  float* C;
  int n, base, sign;
  bool mirror;
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < n && col < n) {
      const int r = base + sign * row, c = base + sign * col;
      C[(size_t)r * n + c] = v;
      if (mirror && row != col) C[(size_t)c * n + r] = v;
    }
  }
};

// dst = Y Y^T over the upper tiles (k >= the later block), mirrored
__global__ __launch_bounds__(NTHREADS) void lauum_kernel(const MatDesc* table, const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  if (m.noinv) return;
  int bi, bj;
  lauum_tile(m.T, local, bi, bj);
  const int n = m.n;
  DenseMK P{m.Y, n, n};
  EpiSymFlip epi{m.U, n, m.rev ? n - 1 : 0, m.rev ? -1 : 1, bi != bj};
  gemm_tile(P, P, bi * BM, bj * BN, bj * DB, n, bi == bj, epi, smem);
}

// W = J Y^T J (J = reversal) for the matrices factored back to front: with S = J X J = R^T R
// and Y = R^-1, X^-1 = J Y Y^T J = W^T W and W is upper triangular with a positive diagonal,
// i.e. the upper Cholesky factor of X^-1, read off the triangular inverse instead of being
// computed by a second factorisation.  W[i][j] = Y[n-1-j][n-1-i] for j >= i, 0 below;
// 64 x 64 tiles through LDS so that reads and writes are both row-contiguous.
__global__ __launch_bounds__(256) void std_from_inverse_factor_kernel(const MatDesc* table,
                                                                      const WorkList wl) {
  __shared__ float tile[64][65];
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  if (m.W == nullptr) return;
  const int n = m.n;
  const int T64 = (n + 63) / 64;
  const int ti = local / T64, tj = local - ti * T64;       // tile of W: rows ti, columns tj
  const int i0 = ti * 64, j0 = tj * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (tj >= ti) {
    // source element for W[i0 + a][j0 + b] is Y[n-1-j0-b][n-1-i0-a]: lanes run along a
    for (int b = ty; b < 64; b += 4) {
      const int r = n - 1 - j0 - b, c = n - 1 - i0 - tx;
      tile[b][tx] = (r >= 0 && c >= 0 && c >= r) ? m.Y[(size_t)r * n + c] : 0.f;
    }
  }
  __syncthreads();
  for (int a = ty; a < 64; a += 4) {
    const int i = i0 + a, j = j0 + tx;
    if (i < n && j < n) m.W[(size_t)i * n + j] = (tj >= ti && j >= i) ? tile[tx][a] : 0.f;
  }
}

// zero the strictly lower triangle of a triangular result: of U for every matrix
// (Cholesky-factor output), or, with `of_y`, of Y for the matrices whose result Y is
__global__ __launch_bounds__(256) void zero_lower_kernel(const MatDesc* table, int of_y,
                                                         const WorkList wl) {
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  if (of_y && !m.noinv) return;
  float* const X = of_y ? m.Y : m.U;
  const int n = m.n;
  const int T = m.T;
  const int bi = local / T, bj = local - bi * T;
  if (bj > bi) return;
  for (int e = threadIdx.x; e < BM * BN; e += 256) {
    const int row = bi * BM + (e >> 7);
    const int col = bj * BN + (e & 127);
    if (row < n && col < n && col < row) X[(size_t)row * n + col] = 0.f;
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct HostMat {
  const float* src;
  float* dst;
  int n;
  float damp;
  int partner;   // index in caller order, or -1
  int is_a;
  int out;
  float* std = nullptr;   // non-null: factor back to front and also deliver the upper
                          // Cholesky factor W of the inverse (W^T W = inverse; the posterior
                          // std of Noisy K-FAC)
  float* fac = nullptr;   // non-null (then dst and std are null): deliver the inverse as its
                          // triangular factor only, Y upper with Y Y^T = inverse
};

static size_t inverse_workspace_bytes(const std::vector<int>& dims) {
  size_t bytes = align256(dims.size() * sizeof(MatDesc));
  for (int n : dims) bytes += align256((size_t)n * n * sizeof(float));
  return bytes;
}

enum { MODE_INVERSE = 0, MODE_CHOLESKY = 1 };

static int run_batched(std::vector<HostMat>& mats, int mode, int* info, void* workspace,
                       size_t workspace_bytes, hipStream_t stream) {
  const int nmat = (int)mats.size();
  if (nmat == 0) return KFAC_OK;
  std::vector<int> dims(nmat);
  for (int i = 0; i < nmat; ++i) dims[i] = mats[i].n;
  if (workspace == nullptr || workspace_bytes < inverse_workspace_bytes(dims))
    return KFAC_ERR_WORKSPACE;

  // kernels that need more than the default 64 KiB of LDS (registered once per process)
  if (!enable_large_lds((const void*)potrf_diag_kernel, DIAG_SMEM_BYTES) ||
      !enable_large_lds((const void*)potrf_step_kernel, DIAG_SMEM_BYTES) ||
      !enable_large_lds((const void*)potrf_fine_kernel, FINE_SMEM_BYTES) ||
      !enable_large_lds((const void*)potrf_sub_kernel, SUB_SMEM_BYTES))
    return KFAC_ERR_LAUNCH;

  // descending size order; remember where each caller index went
  std::vector<int> order(nmat);
  for (int i = 0; i < nmat; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(),
                   [&](int a, int b) { return mats[a].n > mats[b].n; });
  std::vector<int> pos(nmat);
  for (int s = 0; s < nmat; ++s) pos[order[s]] = s;

  MatDesc* table = (MatDesc*)workspace;
  char* ybase = (char*)workspace + align256(nmat * sizeof(MatDesc));
  size_t yoff = 0;
  int Tmax = 0;
  std::vector<int> Ts(nmat);
  for (int s0 = 0; s0 < nmat; s0 += SETUP_CHUNK) {
    DescChunk chunk;
    const int cnt = std::min(SETUP_CHUNK, nmat - s0);
    for (int k = 0; k < cnt; ++k) {
      const HostMat& h = mats[order[s0 + k]];
      MatDesc& d = chunk.d[k];
      d.src = h.src;
      // the slot of the workspace holds Y, or, when Y goes straight to the caller, the
      // Cholesky factor that nobody asked for
      d.noinv = h.fac != nullptr;
      d.pad = 0;
      d.U = d.noinv ? (float*)(ybase + yoff) : h.dst;
      d.Y = d.noinv ? h.fac : (float*)(ybase + yoff);
      yoff += align256((size_t)h.n * h.n * sizeof(float));
      d.n = h.n;
      d.T = cdiv(h.n, DB);
      d.damp = h.damp;
      d.partner = h.partner < 0 ? -1 : pos[h.partner];
      d.is_a = h.is_a;
      d.out = h.out;
      d.trace = 0.f;
      d.rev = h.std != nullptr;
      d.W = h.std;
      Ts[s0 + k] = d.T;
      Tmax = std::max(Tmax, d.T);
    }
    hipLaunchKernelGGL(inv_setup_kernel, dim3(1), dim3(SETUP_CHUNK), 0, stream, chunk, table, s0,
                       cnt);
  }
  auto active = [&](int minT) {   // matrices with T >= minT (a prefix of the sorted table)
    int c = 0;
    while (c < nmat && Ts[c] >= minT) ++c;
    return c;
  };

  // Runs `launch(worklist)` over the first `count` matrices of the sorted table,
  // WL_MAX at a time, with items(T) work items for a matrix of T blocks; matrices
  // without items are skipped at the ends and cost nothing in between.
  auto for_worklists = [&](int count, auto&& items, auto&& launch) {
    for (int s0 = 0; s0 < count; s0 += WL_MAX) {
      WorkList wl;
      wl.first = s0;
      wl.n = std::min(WL_MAX, count - s0);
      wl.cum[0] = 0;
      for (int i = 0; i < wl.n; ++i) wl.cum[i + 1] = wl.cum[i] + std::max(0, (int)items(Ts[s0 + i]));
      for (int i = wl.n + 1; i <= WL_MAX; ++i) wl.cum[i] = wl.cum[wl.n];
      if (wl.cum[wl.n] > 0) launch(wl, wl.cum[wl.n]);
    }
  };

  bool any_pi = false;
  for (auto& h : mats) any_pi |= h.partner >= 0;
  if (any_pi) hipLaunchKernelGGL(inv_trace_kernel, dim3(nmat), dim3(256), 0, stream, table);
  for_worklists(nmat, [](int T) { return T * (T + 1) / 2; }, [&](const WorkList& wl, int grid) {
    hipLaunchKernelGGL(inv_copy_damp_kernel, dim3(grid), dim3(256), 0, stream, table, info, wl);
  });

  for (int P0 = 0, Pend = 0; P0 < Tmax; P0 = Pend) {
    Pend = Tmax - P0 <= TAIL_BLOCKS ? Tmax : std::min(P0 + GROUP_BLOCKS, Tmax);
    auto total_items = [&](int count, auto&& items) {
      long sum = 0;
      for (int i = 0; i < count; ++i) sum += std::max(0, (int)items(Ts[i]));
      return sum;
    };
    for (int p = P0; p < Pend; ++p) {
      const int na = active(p + 1);
      // diagonal block p; from the group's second block on it first takes panel p-1's update
      // itself, and the same launch holds the tiles that apply that panel to the other rows
      // of the group (block row p first: the next row panel needs it; nothing else needs any
      // of them before the next launch)
      auto rest_items = [&](int T) {
        const int Tr = T - p;          // (all remaining rows: the upper triangle of tiles)
        return Pend >= T ? Tr * (Tr + 1) / 2 : (Pend - p) * Tr;
      };
      if (p == P0) {
        hipLaunchKernelGGL(potrf_diag_kernel, dim3(na), dim3(DIAG_THREADS), DIAG_SMEM_BYTES, stream,
                           table, p, info);
      } else {
        bool first = true;
        for_worklists(na, rest_items, [&](const WorkList& wl, int grid) {
          const int nd = first ? na : 0;
          first = false;
          // (one workgroup runs per compute unit: beyond 256 tiles, up to three to a workgroup)
          const int tpw = std::min(STEP_TILES_PER_WG, std::max(1, cdiv(grid, 256)));
          hipLaunchKernelGGL(potrf_step_kernel, dim3(nd + cdiv(grid, tpw)), dim3(DIAG_THREADS),
                             DIAG_SMEM_BYTES, stream, table, p, info, nd, p, Pend, tpw, wl);
        });
      }
      const int nb = active(p + 2);
      if (nb == 0) continue;
      auto panel_items = [&](int T) { return T - p - 1; };
      if (total_items(nb, panel_items) <= SUB_MAX_TILES) {
        for_worklists(nb, [&](int T) { return 4 * std::max(0, panel_items(T)); },
                      [&](const WorkList& wl, int grid) {
                        hipLaunchKernelGGL(potrf_sub_kernel, dim3(grid), dim3(SUB_THREADS),
                                           SUB_SMEM_BYTES, stream, table, p, wl);
                      });
      } else
      for_worklists(nb, panel_items, [&](const WorkList& wl, int grid) {
        if (grid <= FINE_MAX_TILES)
          hipLaunchKernelGGL(potrf_fine_kernel, dim3(grid), dim3(FINE_THREADS), FINE_SMEM_BYTES,
                             stream, table, p, wl);
        else
          KFAC_LAUNCH_TILE2(potrf_panel_kernel, dim3(grid), stream, table, p, wl);
      });
    }
    const int nc = active(Pend + 1);
    if (Pend < Tmax && nc > 0) {
      for_worklists(nc, [&](int T) { const int Tr = T - Pend; return Tr * (Tr + 1) / 2; },
                    [&](const WorkList& wl, int grid) {
                      KFAC_LAUNCH_TILE2(potrf_trail_kernel, dim3(grid), stream, table, P0,
                                        Pend - P0, Pend, Tmax, wl);
                    });
    }
  }
  if (mode == MODE_CHOLESKY) {
    for_worklists(nmat, [](int T) { return T * T; }, [&](const WorkList& wl, int grid) {
      hipLaunchKernelGGL(zero_lower_kernel, dim3(grid), dim3(256), 0, stream, table, 0, wl);
    });
    return launch_status();
  }
  if (Tmax > 1) {
    int D = 0;
    while ((1 << D) < Tmax) ++D;
    const int na = active(2);
    for (int depth = D - 1; depth >= 0 && na > 0; --depth) {
      // matrices with fewer than 2^depth blocks have no merge this deep
      auto pairs = [&](int T) { return (1 << depth) < T ? merge_tiles(T, depth) : 0; };
      for_worklists(na, pairs, [&](const WorkList& wl, int grid) {
        KFAC_LAUNCH_TILE2(trtri_w_kernel, dim3(grid), stream, table, depth, wl);
      });
      for_worklists(na, pairs, [&](const WorkList& wl, int grid) {
        KFAC_LAUNCH_TILE2(trtri_y_kernel, dim3(grid), stream, table, depth, wl);
      });
    }
  }
  bool any_inv = false, any_std = false, any_fac = false;
  for (auto& h : mats) {
    any_inv |= h.dst != nullptr;
    any_std |= h.std != nullptr;
    any_fac |= h.fac != nullptr;
  }
  if (any_inv)
    for_worklists(nmat, [](int T) { return T * (T + 1) / 2; }, [&](const WorkList& wl, int grid) {
      KFAC_LAUNCH_TILE2(lauum_kernel, dim3(grid), stream, table, wl);
    });
  if (any_fac)   // the triangular inversion kept intermediate products below the diagonal
    for_worklists(nmat, [](int T) { return T * T; }, [&](const WorkList& wl, int grid) {
      hipLaunchKernelGGL(zero_lower_kernel, dim3(grid), dim3(256), 0, stream, table, 1, wl);
    });
  if (any_std) {
    // (items per matrix: its 64 x 64 tiles; Ts holds 128-blocks, so 4 T^2 covers them)
    for_worklists(nmat, [](int T) { return 4 * T * T; }, [&](const WorkList& wl, int grid) {
      hipLaunchKernelGGL(std_from_inverse_factor_kernel, dim3(grid), dim3(256), 0, stream, table,
                         wl);
    });
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// Scratch for the entry point that allocates nothing: one array in device memory,
// part of the code object, so every GPU this library runs on holds its own copy at
// its own address until the process ends.  In host code the name `scratch` is only a
// handle for hipGetSymbolAddress; kernels and memory calls get the address it returns.
// ---------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int SCRATCH_MAX_DEVICES = 64;
static std::atomic<void*> scratch_ptr[SCRATCH_MAX_DEVICES];   // address on each device, once known

// Device address of `scratch` on the current device (looked up on the first call on that
// device); nullptr on failure.
static void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEVICES) return nullptr;
  void* ptr = scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr != nullptr) return ptr;
  if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr)
    return nullptr;
  scratch_ptr[dev].store(ptr, std::memory_order_release);
  return ptr;
}

// Calls that share the array are put in order: each call records an event behind its last
// kernel, and the next call on that device makes its stream wait for it first (a no-op for
// the single-stream caller).  The events are created on a device's first call.  A stream
// under graph capture takes no part: an event recorded outside a capture cannot be waited
// for inside one, and inside a graph the graph's own order applies.
static std::mutex scratch_mutex;
static hipEvent_t scratch_done[SCRATCH_MAX_DEVICES];    // (never destroyed: no teardown order)
static bool scratch_done_set[SCRATCH_MAX_DEVICES];

static bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

}  // namespace kfac

using namespace kfac;

extern "C" {

size_t kfac_static_workspace_bytes(void) { return STATIC_SCRATCH_BYTES; }

int kfac_damped_inverse_batched_static(int count, const int* dims, const float* const* src,
                                       const float* damp, float* const* dst, int* info,
                                       void* stream) {
  if (count < 0 || (count > 0 && (!dims || !src || !dst || !info))) return KFAC_ERR_ARG;
  std::vector<HostMat> mats(count);
  std::vector<int> d(count);
  for (int i = 0; i < count; ++i) {
    if (dims[i] <= 0 || dims[i] > 16384 || !src[i] || !dst[i] || src[i] == dst[i])
      return KFAC_ERR_ARG;
    mats[i] = HostMat{src[i], dst[i], dims[i], damp ? damp[i] : 0.f, -1, 0, i};
    d[i] = dims[i];
  }
  if (count == 0) return KFAC_OK;
  if (inverse_workspace_bytes(d) > STATIC_SCRATCH_BYTES) return KFAC_ERR_TOO_LARGE;
  void* ptr = static_scratch();
  if (ptr == nullptr) return KFAC_ERR_LAUNCH;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEVICES) return KFAC_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> order(scratch_mutex);
  const bool ordered = !stream_is_capturing(st);
  if (ordered) {
    if (!scratch_done_set[dev]) {
      if (hipEventCreateWithFlags(&scratch_done[dev], hipEventDisableTiming) != hipSuccess)
        return KFAC_ERR_LAUNCH;
      scratch_done_set[dev] = true;
    } else if (hipStreamWaitEvent(st, scratch_done[dev], 0) != hipSuccess) {
      return KFAC_ERR_LAUNCH;
    }
  }
  const int status = run_batched(mats, MODE_INVERSE, info, ptr, STATIC_SCRATCH_BYTES, st);
  if (ordered && hipEventRecord(scratch_done[dev], st) != hipSuccess) return KFAC_ERR_LAUNCH;
  return status;
}

double kfac_inverse_executed_flops(int count, const int* dims, const int* factored) {
  if (count <= 0 || !dims) return 0.;
  const double B = 2. * DB * DB * DB;       // one 128-deep step of a 128 x 128 tile
  // diagonal block: per strip 4 waves x 15 rank-2 steps x 2 blocks, the updates by finished
  // strips (12 + 8 blocks, 32 deep), the pending panel (10 blocks, 128 deep)
  const double diag = 4096. * (4 * 120 + 20 * 16 + 10 * 64);
  double total = 0.;
  for (int i = 0; i < count; ++i) {
    const double T = cdiv(dims[i], DB);
    // Cholesky: row panels, trailing updates (whole diagonal tiles)
    total += T * diag + B * (T * (T - 1) / 2 + (T - 1) * T * (T + 1) / 6);
    // triangular inverse: per merge of r x c blocks, W tiles reduce over 1..c blocks,
    // Y tiles over r..1
    const int Ti = (int)T;
    int D = 0;
    while ((1 << D) < Ti) ++D;
    for (int depth = 0; depth < D; ++depth)
      for (int P = 0; P < (1 << depth); ++P) {
        const Segment sg = segment(P, depth, Ti);
        const double r = sg.mid - sg.p0, c = sg.p1 - sg.mid;
        total += B * (r * c * (c + 1) / 2 + c * r * (r + 1) / 2);
      }
    // Y Y^T where the explicit inverse is formed: tile (bi <= bj) reduces over T - bj blocks
    if (!(factored && factored[i]))
      for (int bj = 0; bj < Ti; ++bj) total += B * (bj + 1.) * (T - bj);
  }
  return total;
}

size_t kfac_inverse_workspace_bytes(int count, const int* dims) {
  if (count <= 0 || !dims) return 0;
  std::vector<int> d(dims, dims + count);
  for (int n : d)
    if (n <= 0) return 0;
  return inverse_workspace_bytes(d);
}

int kfac_damped_inverse_batched(int count, const int* dims, const float* const* src,
                                const float* damp, float* const* dst, int* info,
                                void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!dims || !src || !dst || !info))) return KFAC_ERR_ARG;
  std::vector<HostMat> mats(count);
  for (int i = 0; i < count; ++i) {
    if (dims[i] <= 0 || dims[i] > 16384 || !src[i] || !dst[i] || src[i] == dst[i])
      return KFAC_ERR_ARG;
    mats[i] = HostMat{src[i], dst[i], dims[i], damp ? damp[i] : 0.f, -1, 0, i};
  }
  return run_batched(mats, MODE_INVERSE, info, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_pi_damped_inverse_batched(int layers, const int* dA, const int* dG,
                                   const float* const* A, const float* const* G,
                                   const float* damping, float* const* Ainv, float* const* Ginv,
                                   int* info, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  if (layers < 0 || (layers > 0 && (!dA || !dG || !A || !G || !damping || !Ainv || !Ginv || !info)))
    return KFAC_ERR_ARG;
  std::vector<HostMat> mats(2 * layers);
  for (int l = 0; l < layers; ++l) {
    if (dA[l] <= 0 || dG[l] <= 0 || dA[l] > 16384 || dG[l] > 16384 || !A[l] || !G[l] ||
        !Ainv[l] || !Ginv[l] || A[l] == Ainv[l] || G[l] == Ginv[l] || !(damping[l] >= 0.f))
      return KFAC_ERR_ARG;
    const float r = sqrtf(damping[l]);
    mats[2 * l] = HostMat{A[l], Ainv[l], dA[l], r, 2 * l + 1, 1, 2 * l};
    mats[2 * l + 1] = HostMat{G[l], Ginv[l], dG[l], r, 2 * l, 0, 2 * l + 1};
  }
  return run_batched(mats, MODE_INVERSE, info, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_pi_damped_inverse_std_batched(int layers, const int* dA, const int* dG,
                                       const float* const* A, const float* const* G,
                                       const float* damping, float* const* Ainv,
                                       float* const* Ginv, float* const* Astd,
                                       float* const* Gstd, int* info, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  if (layers < 0 || (layers > 0 && (!dA || !dG || !A || !G || !damping || !Ainv || !Ginv ||
                                    !Astd || !Gstd || !info)))
    return KFAC_ERR_ARG;
  std::vector<HostMat> mats(2 * layers);
  for (int l = 0; l < layers; ++l) {
    if (dA[l] <= 0 || dG[l] <= 0 || dA[l] > 16384 || dG[l] > 16384 || !A[l] || !G[l] ||
        !Ainv[l] || !Ginv[l] || A[l] == Ainv[l] || G[l] == Ginv[l] || !(damping[l] >= 0.f))
      return KFAC_ERR_ARG;
    if (Astd[l] && (Astd[l] == Ainv[l] || Astd[l] == A[l])) return KFAC_ERR_ARG;
    if (Gstd[l] && (Gstd[l] == Ginv[l] || Gstd[l] == G[l])) return KFAC_ERR_ARG;
    const float r = sqrtf(damping[l]);
    mats[2 * l] = HostMat{A[l], Ainv[l], dA[l], r, 2 * l + 1, 1, 2 * l, Astd[l]};
    mats[2 * l + 1] = HostMat{G[l], Ginv[l], dG[l], r, 2 * l, 0, 2 * l + 1, Gstd[l]};
  }
  return run_batched(mats, MODE_INVERSE, info, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_pi_damped_inverse_factored_batched(int layers, const int* dA, const int* dG,
                                            const float* const* A, const float* const* G,
                                            const float* damping, float* const* Ainv,
                                            float* const* Ginv, float* const* Afac,
                                            float* const* Gfac, int* info, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  if (layers < 0 || (layers > 0 && (!dA || !dG || !A || !G || !damping || !Ainv || !Ginv ||
                                    !Afac || !Gfac || !info)))
    return KFAC_ERR_ARG;
  std::vector<HostMat> mats(2 * layers);
  for (int l = 0; l < layers; ++l) {
    if (dA[l] <= 0 || dG[l] <= 0 || dA[l] > 16384 || dG[l] > 16384 || !A[l] || !G[l] ||
        !(damping[l] >= 0.f))
      return KFAC_ERR_ARG;
    // per matrix exactly one of the two forms, never on top of its input
    if ((Ainv[l] == nullptr) == (Afac[l] == nullptr) || (Ginv[l] == nullptr) == (Gfac[l] == nullptr))
      return KFAC_ERR_ARG;
    if (Ainv[l] == A[l] || Afac[l] == A[l] || Ginv[l] == G[l] || Gfac[l] == G[l])
      return KFAC_ERR_ARG;
    const float r = sqrtf(damping[l]);
    mats[2 * l] = HostMat{A[l], Ainv[l], dA[l], r, 2 * l + 1, 1, 2 * l, nullptr, Afac[l]};
    mats[2 * l + 1] = HostMat{G[l], Ginv[l], dG[l], r, 2 * l, 0, 2 * l + 1, nullptr, Gfac[l]};
  }
  return run_batched(mats, MODE_INVERSE, info, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_cholesky_upper_batched(int count, const int* dims, const float* const* src,
                                float* const* dst, int* info, void* workspace,
                                size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!dims || !src || !dst || !info))) return KFAC_ERR_ARG;
  std::vector<HostMat> mats(count);
  for (int i = 0; i < count; ++i) {
    if (dims[i] <= 0 || dims[i] > 16384 || !src[i] || !dst[i] || src[i] == dst[i])
      return KFAC_ERR_ARG;
    mats[i] = HostMat{src[i], dst[i], dims[i], 0.f, -1, 0, i};
  }
  return run_batched(mats, MODE_CHOLESKY, info, workspace, workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
