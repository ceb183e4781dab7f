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
//      update at once (the next row before anything else, the others from tile
//      workgroups that share a launch with the next diagonal block, so that the
//      chip is not idle while that latency-bound block is factored), the rows
//      beyond the group receive the whole group in one deeper product;
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
constexpr int WLD = 65;
constexpr int DIAG_SMEM_BYTES = (2 * DB * DLD + 64 * WLD) * (int)sizeof(float);

// One wave runs the 32 elimination steps of the 32-row strip at row c0 of S on two
// column blocks at once: lanes 0-31 hold the columns of the diagonal leaf
// (c0 .. c0+31), lanes 32-63 the columns pcol .. pcol+31 of the same rows (a
// block of the row panel to the right; pcol < 0: none, the lanes shadow the leaf).
// Lane j keeps its column in registers.  Each step needs row c of the leaf in every
// lane: the leaf lanes write their element to a 64-float LDS buffer private to
// the wave and all lanes read the row back with broadcast ds_read_b128.  The steps
// are software-pipelined: step c first finishes element c+1 of the column, publishes
// it (two buffers alternate) and issues the reads of row c+1, and only then applies
// row c to the rest of the column, so the LDS round trip of the next row runs under
// those FMAs (scheduling barriers keep the compiler from moving them in front of the
// store); the pivot itself comes through v_readlane and does not wait for LDS.
// The panel columns see the same eliminations as the leaf columns, so the strip ends
// up holding U[q][*] without a triangular solve.  Several waves may run this on the
// same leaf with different panel blocks (the leaf is then factored redundantly; only
// `owner` writes it out, as a dense 32x32 copy `ubuf`, which the caller copies over
// the leaf in S once all waves are past reading it, and which feeds the back
// substitution).
__device__ __forceinline__ float lane_value(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src_lane));
}

__device__ __forceinline__ void read_row(const lds_f* rowbuf, int first, float (&row)[32]) {
#pragma unroll
  for (int g = first / 4; g < 8; ++g) {
    const v4f v = *(const lds_f4*)(rowbuf + 4 * g);
    row[4 * g + 0] = v.x;
    row[4 * g + 1] = v.y;
    row[4 * g + 2] = v.z;
    row[4 * g + 3] = v.w;
  }
}

__device__ __forceinline__ void chol_strip_32(lds_f* S, lds_f* rowbuf, lds_f* ubuf, int c0,
                                              int pcol, bool owner, int row_base, int* info) {
  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const bool leaf = lane < 32;
  const int col = (leaf || pcol < 0) ? c0 + j : pcol + j;
  float a[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) a[i] = S[(c0 + i) * DLD + col];
  int bad = 0;
  // A[c][c0 + j] after the updates of the earlier steps; the panel lanes write into
  // the unused second half of the buffer, so that the store is unconditional
  float row[32];
  rowbuf[lane] = a[0];
  __builtin_amdgcn_wave_barrier();
  read_row(rowbuf, 0, row);
  float piv = lane_value(a[0], 0);
  // 1/sqrt in one instruction: the next step's pivot waits on this chain
  float rd = __builtin_amdgcn_rsqf(piv);
  float f = a[0] * (rd * rd);
#pragma unroll
  for (int c = 0; c < 32; ++c) {
    if (!(piv > 0.f) && bad == 0) bad = row_base + c0 + c + 1;
    float next[32];
    float pivn = 0.f, rdn = 0.f, fn = 0.f;
    if (c + 1 < 32) {
      // the chain from step to step: element c+1, its store, the reads of row c+1
      a[c + 1] = fmaf(-row[c + 1], f, a[c + 1]);
      lds_f* const nb = rowbuf + 64 * ((c + 1) & 1);
      nb[lane] = a[c + 1];
      __builtin_amdgcn_wave_barrier();
      read_row(nb, c + 1, next);
      // nothing may be scheduled in front of that store: the rest of this step is
      // what runs while the row travels through LDS
      __builtin_amdgcn_sched_barrier(0);
      pivn = lane_value(a[c + 1], c + 1);
      rdn = __builtin_amdgcn_rsqf(pivn);
      fn = a[c + 1] * (rdn * rdn);
    }
#pragma unroll
    for (int i = c + 2; i < 32; ++i) a[i] = fmaf(-row[i], f, a[i]);   // A[i][col] -= U[c][i] U[c][col]
    const float u = a[c] * rd;
    a[c] = leaf ? (j > c ? u : (j == c ? piv * rd : 0.f)) : u;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = c + 1; i < 32; ++i) row[i] = next[i];
    piv = pivn;
    rd = rdn;
    f = fn;
  }
  if (owner && bad != 0 && lane == 0) {
    if (*info == 0) *info = bad;
  }
  if (leaf) {
    if (owner) {
#pragma unroll
      for (int i = 0; i < 32; ++i) ubuf[i * 32 + j] = (i <= j) ? a[i] : 0.f;
    }
  } else if (pcol >= 0) {
#pragma unroll
    for (int i = 0; i < 32; ++i) S[(c0 + i) * DLD + pcol + j] = a[i];
  }
}

// One wave: Y = U^-1 of the 32x32 upper-triangular leaf in ubuf (dense, row-major),
// written to Yb at (c0, c0).  Column j of Y in lane j, row i of U broadcast.
__device__ __forceinline__ void backsub_32(const lds_f* ubuf, lds_f* Yb, int c0) {
  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  float y[32];
#pragma unroll
  for (int i = 31; i >= 0; --i) {
    float row[32];
#pragma unroll
    for (int g = i / 4; g < 8; ++g) {
      const v4f v = *(const lds_f4*)(ubuf + i * 32 + 4 * g);
      row[4 * g + 0] = v.x;
      row[4 * g + 1] = v.y;
      row[4 * g + 2] = v.z;
      row[4 * g + 3] = v.w;
    }
    // y[i+1] was finished last: it enters the sum last, so that only one FMA and
    // one multiply separate consecutive rows; two partial sums shorten the rest
    float s0 = (j == i) ? 1.f : 0.f, s1 = 0.f;
#pragma unroll
    for (int k = 31; k > i + 1; k -= 2) {
      s0 = fmaf(-row[k], y[k], s0);
      if (k - 1 > i + 1) s1 = fmaf(-row[k - 1], y[k - 1], s1);
    }
    float s = s0 + s1;
    if (i + 1 < 32) s = fmaf(-row[i + 1], y[i + 1], s);
    y[i] = s * __builtin_amdgcn_rcpf(row[i]);
  }
  if (lane < 32) {
#pragma unroll
    for (int i = 0; i < 32; ++i) Yb[(c0 + i) * DLD + c0 + j] = (i <= j) ? y[i] : 0.f;
  }
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
  // 32 deep at a time: the 32 operand reads are issued together, ahead of the 16 MFMAs
  for (int k0 = 0; k0 < K; k0 += 32) {
    float av[16], bv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      av[i] = pa[(k0 + 2 * i) * a_ks];
      bv[i] = pb[(k0 + 2 * i) * b_ks];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[i], acc, 0, 0, 0);
  }
  return acc;
}

// store / subtract a 32x32 result block at c[row*ld + col]
__device__ __forceinline__ void lds_put32(lds_f* c, int ld, const v16f& acc, float scale) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
#pragma unroll
  for (int t = 0; t < 16; ++t) c[(8 * (t >> 2) + 4 * h + (t & 3)) * ld + r] = scale * acc[t];
}
__device__ __forceinline__ void lds_sub32(lds_f* c, int ld, const v16f& acc) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
#pragma unroll
  for (int t = 0; t < 16; ++t) c[(8 * (t >> 2) + 4 * h + (t & 3)) * ld + r] -= acc[t];
}

// In-LDS off-diagonal inverse block:  Y12 = -Y11 * (U12 * Y22) for the pair
// X1 = [s1, s1+b), X2 = [s1+b, s1+2b), b = 32 or 64; W is a b x b scratch.
// 32x32 result blocks are dealt round-robin to the 4 waves.
__device__ __forceinline__ void tri_pair(const lds_f* S, lds_f* Yb, lds_f* Wt, int s1, int b,
                                         int wave_first, int wave_count) {
  const int s2 = s1 + b;
  const int wave = (int)(threadIdx.x >> 6) - wave_first;
  const int nb = b / 32;
  // W[i][j] = sum_k U12[i][k] * Y22[k][j]     (Y22 is zero below its diagonal)
  for (int blk = wave; blk < nb * nb && wave >= 0; blk += wave_count) {
    const int bi = blk / nb, bj = blk - bi * nb;
    const v16f acc = lds_mma32(S + (s1 + 32 * bi) * DLD + s2, 1, DLD,
                               Yb + s2 * DLD + s2 + 32 * bj, DLD, 1, 32 * (bj + 1));
    lds_put32(Wt + 32 * bi * WLD + 32 * bj, WLD, acc, 1.f);
  }
  __syncthreads();
  // Y12[i][j] = - sum_{k} Y11[i][k] * W[k][j]  (Y11 is zero below its diagonal)
  for (int blk = wave; blk < nb * nb && wave >= 0; blk += wave_count) {
    const int bi = blk / nb, bj = blk - bi * nb;
    const v16f acc = lds_mma32(Yb + (s1 + 32 * bi) * DLD + s1 + 32 * bi, 1, DLD,
                               Wt + 32 * bi * WLD + 32 * bj, WLD, 1, b - 32 * bi);
    lds_put32(Yb + (s1 + 32 * bi) * DLD + s2 + 32 * bj, DLD, acc, -1.f);
  }
  __syncthreads();
}

// Factors and inverts diagonal block p of matrix m (one workgroup of 256 threads with
// DIAG_SMEM_BYTES of LDS at dsm).
__device__ __forceinline__ void diag_block(const MatDesc& m, int p, int* info, float* dsm) {
  lds_f* const S = (lds_f*)dsm;
  lds_f* const Yb = S + DB * DLD;
  lds_f* const Wt = S + 2 * DB * DLD;
  const int n = m.n;
  const int r0 = p * DB;
  const int nb = min(DB, n - r0);
  const int t = threadIdx.x;
  const int wave = t >> 6;

  // load the upper triangle; pad with the identity up to 128.  32 loads are
  // issued before the first is used, so the block costs 2 memory round trips
  // instead of 64.
  // (raw buffer loads: no 64-bit address per element, and the elements outside the
  // triangle cost no memory access)
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(m.U + (size_t)r0 * n + r0);
  for (int e0 = 0; e0 < DB * DB; e0 += 256 * 32) {
    float v[32];
#pragma unroll
    for (int u = 0; u < 32; ++u) {
      const int e = e0 + u * 256 + t;
      const int i = e >> 7, j = e & 127;
      const bool in = i < nb && j < nb && j >= i;
      v[u] = buffer_load(rs, in ? (unsigned)(i * n + j) * 4u : INV_M);
    }
#pragma unroll
    for (int u = 0; u < 32; ++u) {
      const int e = e0 + u * 256 + t;
      const int i = e >> 7, j = e & 127;
      const bool in = i < nb && j < nb && j >= i;
      const bool pad = (i >= nb || j >= nb) && i == j;
      S[i * DLD + j] = in ? v[u] : (pad ? 1.f : 0.f);
      Yb[i * DLD + j] = 0.f;
    }
  }
  __syncthreads();

  // Scratch (in Wt, free until the doubling below): two 64-float row buffers per
  // wave and two dense leaf copies, used alternately.
  lds_f* const rowbuf = Wt + 128 * wave;
  lds_f* const ubuf0 = Wt + 512;
  const int nq = (nb + 31) / 32;
  // One more turn than there are leaves: the last one only inverts the last leaf
  // (a second call site would be a second copy of that code, fetched cold).
  for (int q = 0; q <= nq; ++q) {
    const int c0 = 32 * q;
    const int rest = nq - q - 1;     // 32-blocks to the right
    if (wave < 3) {
      // waves 0..2: the strip of leaf q, each with one block of the row panel
      if (q < nq && (wave == 0 || wave < rest))
        chol_strip_32(S, rowbuf, ubuf0 + 1024 * (q & 1), c0, wave < rest ? c0 + 32 * (wave + 1) : -1,
                      wave == 0, r0, info + m.out);
    } else if (q > 0) {
      // wave 3, meanwhile: inverse of the previous leaf (off the critical path)
      backsub_32(ubuf0 + 1024 * ((q - 1) & 1), Yb, c0 - 32);
    }
    __syncthreads();
    if (q == nq) break;
    if (wave == 0 && (t & 32) == 0) {
      // the factored leaf replaces A[q][q] now that no wave reads the original any more
      const lds_f* ub = ubuf0 + 1024 * (q & 1);
#pragma unroll
      for (int i = 0; i < 32; ++i) S[(c0 + i) * DLD + c0 + t] = ub[i * 32 + t];
    }
    if (rest > 0) {
      // trailing update: A[i][j] -= U[q][i]^T U[q][j], q < i <= j
      const int nblk = rest * (rest + 1) / 2;
      for (int blk = wave; blk < nblk; blk += 4) {
        int bi, bj;
        upper_tile(blk, rest, bi, bj);
        const int ci = c0 + 32 * (bi + 1), cj = c0 + 32 * (bj + 1);
        const v16f acc = lds_mma32(S + c0 * DLD + ci, DLD, 1, S + c0 * DLD + cj, DLD, 1, 32);
        lds_sub32(S + ci * DLD + cj, DLD, acc);
      }
      __syncthreads();
    }
  }

  // inverse of the whole block by doubling: 32 -> 64 -> 128
  if (nq > 1) {
    // the two level-32 pairs use disjoint data: waves 0-1 take the first, 2-3 the second
    // (both calls contain the same two barriers, reached by every wave)
    if (nq > 3) {
      const int s1 = wave < 2 ? 0 : 64;
      tri_pair(S, Yb, Wt + (wave < 2 ? 0 : 32 * WLD), s1, 32, wave < 2 ? 0 : 2, 2);
    } else {
      tri_pair(S, Yb, Wt, 0, 32, 0, 4);
    }
  }
  if (nq > 2) tri_pair(S, Yb, Wt, 0, 64, 0, 4);

  // write U_pp and Y_pp back, 16 LDS reads in flight per thread
  typedef __attribute__((address_space(1))) float global_f;
  global_f* const gU = (global_f*)(m.U + (size_t)r0 * n + r0);
  global_f* const gY = (global_f*)(m.Y + (size_t)r0 * n + r0);
  for (int e0 = 0; e0 < DB * DB; e0 += 256 * 16) {
    float u[16], y[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int e = e0 + k * 256 + t;
      const int i = e >> 7, j = e & 127;
      u[k] = S[i * DLD + j];
      y[k] = Yb[i * DLD + j];
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int e = e0 + k * 256 + t;
      const int i = e >> 7, j = e & 127;
      if (i < nb && j < nb) {
        gU[i * n + j] = u[k];
        gY[i * n + j] = y[k];
      }
    }
  }
}

__global__ __launch_bounds__(256) void potrf_diag_kernel(const MatDesc* table, int p, int* info) {
  extern __shared__ __attribute__((aligned(16))) float dsm[];
  diag_block(table[blockIdx.x], p, info, dsm);
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
// the others one tile each.  The launch carries the diagonal block's LDS, so one
// workgroup runs per CU: the tile workgroups use the CUs that the few diagonal blocks
// leave idle, for about as long as a diagonal block takes.
__global__ __launch_bounds__(NTHREADS) void potrf_step_kernel(const MatDesc* table, int p,
                                                              int* info, int ndiag, int row_lo,
                                                              int row_hi, const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float dsm[];
  if ((int)blockIdx.x < ndiag) {
    diag_block(table[blockIdx.x], p, info, dsm);
    return;
  }
  int mat, local;
  work_find_item(wl, (int)blockIdx.x - ndiag, mat, local);
  const MatDesc m = table[mat];
  int bi, bj;
  if (!trail_tile(m.T, row_lo, row_hi, local, bi, bj)) return;
  const int n = m.n;
  DenseKM P{m.U + (size_t)(p - 1) * DB * n, nullptr, n, n, 0};
  EpiStore epi{m.U, n, n, n, -1.f, 1.f, false};
  gemm_tile(P, P, bi * BM, bj * BN, 0, DB, bi == bj, epi, dsm);
}

// The row panel (near == 0) or the near update with one block row (near == 1) for
// launches of few tiles: the same 128x128x128 product, but by 16 waves with one
// 32x32 block each instead of 4 waves with four.  A tile is a chain of dependent-issue
// MFMAs, 256 per wave (7.8 us) in the tile engine and 64 here, and at the end of a
// factorisation nothing else runs beside it.  Both operands are fetched whole (32
// loads per thread in flight, and the old values of C with them) into 128 KB of LDS.
constexpr int FINE_THREADS = 1024;
constexpr int FINE_SMEM_BYTES = 2 * DB * DB * (int)sizeof(float);
constexpr int FINE_MAX_TILES = 256;      // one workgroup per CU

__global__ __launch_bounds__(FINE_THREADS) void potrf_fine_kernel(const MatDesc* table, int p,
                                                                  int near, int row_hi,
                                                                  const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float fsm[];
  lds_f* const tp = (lds_f*)fsm;
  lds_f* const tq = tp + DB * DB;
  int mat, local;
  work_find(wl, mat, local);
  const MatDesc m = table[mat];
  const int n = m.n;
  int bi, bj;
  if (near) {
    if (!trail_tile(m.T, p + 1, row_hi, local, bi, bj)) return;
  } else {
    bi = p;
    bj = p + 1 + local;
    if (bj >= m.T) return;
  }
  const float* kbase = m.U + (size_t)p * DB * n;            // block row p of U
  // P(k, i), i < pw;  Q(k, j), j < qw;  C[i][j]
  const float* P = near ? kbase + bi * DB : m.Y + (size_t)p * DB * n + p * DB;
  const float* Q = kbase + bj * DB;
  float* C = m.U + (size_t)bi * DB * n + bj * DB;
  const int pw = near ? min(DB, n - bi * DB) : DB;
  const int qw = min(DB, n - bj * DB);
  const bool same = near && bi == bj;
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int r = lane & 31, h = lane >> 5;
  const int wr = wave >> 2, wc = wave & 3;

  {
    const int mm = t & (DB - 1), kq = t >> 7;
    const __amdgpu_buffer_rsrc_t rp = make_rsrc(P), rq = make_rsrc(Q);
    float vp[16], vq[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const unsigned off = (unsigned)((kq + 8 * i) * n + mm) * 4u;
      vp[i] = buffer_load(rp, mm < pw ? off : INV_M);
      vq[i] = same ? 0.f : buffer_load(rq, mm < qw ? off : INV_M);
    }
    float old[16];
    if (near) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = 32 * wr + 8 * (e >> 2) + 4 * h + (e & 3), col = 32 * wc + r;
        old[e] = (row < pw && col < qw) ? C[(size_t)row * n + col] : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      tp[(kq + 8 * i) * DB + mm] = vp[i];
      if (!same) tq[(kq + 8 * i) * DB + mm] = vq[i];
    }
    __syncthreads();
    const v16f acc = lds_mma32(tp + 32 * wr, DB, 1, (same ? tp : tq) + 32 * wc, DB, 1, DB);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = 32 * wr + 8 * (e >> 2) + 4 * h + (e & 3), col = 32 * wc + r;
      if (row < pw && col < qw) C[(size_t)row * n + col] = near ? old[e] - acc[e] : acc[e];
    }
  }
}

// The same products for launches of very few tiles (at most SUB_MAX_TILES): every tile is
// dealt to four workgroups, so that four CUs' matrix cores work on it.  A workgroup
// takes RB x CB blocks of 32x32 (RB * CB == 4) and 8 waves: a wave does one block over
// half of the 128-deep reduction and the halves are added through LDS.  The near update
// is cut into 64x64 quarters (2 x 2 blocks).  The row panel overwrites its own right-hand
// operand, so its pieces must not share columns: four 128x32 column strips (4 x 1 blocks).
constexpr int SUB_THREADS = 512;
constexpr int SUB_SMEM_BYTES = DB * (128 + 32) * (int)sizeof(float);
constexpr int SUB_MAX_TILES = 64;        // 4 workgroups per tile, one workgroup per CU

template <int RB, int CB>
__global__ __launch_bounds__(SUB_THREADS) void potrf_sub_kernel(const MatDesc* table, int p,
                                                                int near, int row_hi,
                                                                const WorkList wl) {
  constexpr int WP = 32 * RB, WQ = 32 * CB;
  static_assert(RB * CB == 4, "a workgroup takes four 32x32 blocks");
  static_assert(DB * (WP + WQ) * (int)sizeof(float) <= SUB_SMEM_BYTES, "LDS");
  extern __shared__ __attribute__((aligned(16))) float fsm[];
  lds_f* const tp = (lds_f*)fsm;
  lds_f* const tq = tp + DB * WP;
  int mat, item;
  work_find(wl, mat, item);
  const int local = item >> 2, sub = item & 3;
  const int si = sub / (4 / CB), sj = sub % (4 / CB);
  const MatDesc m = table[mat];
  const int n = m.n;
  int bi, bj;
  if (near) {
    if (!trail_tile(m.T, p + 1, row_hi, local, bi, bj)) return;
  } else {
    bi = p;
    bj = p + 1 + local;
    if (bj >= m.T) return;
  }
  const float* kbase = m.U + (size_t)p * DB * n;            // block row p of U
  const float* P = near ? kbase + bi * DB : m.Y + (size_t)p * DB * n + p * DB;
  const float* Q = kbase + bj * DB;
  float* C = m.U + (size_t)bi * DB * n + bj * DB;
  const int pw = near ? min(DB, n - bi * DB) : DB;
  const int qw = min(DB, n - bj * DB);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int r = lane & 31, h = lane >> 5;
  const int blk = wave & 3, khalf = wave >> 2;
  const int br = blk / CB, bc = blk % CB;
  const int row0 = WP * si + 32 * br, col0 = WQ * sj + 32 * bc;   // of this wave's block in the tile

  const __amdgpu_buffer_rsrc_t rp = make_rsrc(P), rq = make_rsrc(Q);
  float vp[WP / 4], vq[WQ / 4];
#pragma unroll
  for (int i = 0; i < WP / 4; ++i) {
    const int idx = t + SUB_THREADS * i;
    const int k = idx / WP, col = WP * si + idx % WP;
    vp[i] = buffer_load(rp, col < pw ? (unsigned)(k * n + col) * 4u : INV_M);
  }
#pragma unroll
  for (int i = 0; i < WQ / 4; ++i) {
    const int idx = t + SUB_THREADS * i;
    const int k = idx / WQ, col = WQ * sj + idx % WQ;
    vq[i] = buffer_load(rq, col < qw ? (unsigned)(k * n + col) * 4u : INV_M);
  }
  float old[16];
  if (near && khalf == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = row0 + 8 * (e >> 2) + 4 * h + (e & 3), col = col0 + r;
      old[e] = (row < pw && col < qw) ? C[(size_t)row * n + col] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < WP / 4; ++i) tp[t + SUB_THREADS * i] = vp[i];
#pragma unroll
  for (int i = 0; i < WQ / 4; ++i) tq[t + SUB_THREADS * i] = vq[i];
  __syncthreads();
  const v16f acc = lds_mma32(tp + 64 * khalf * WP + 32 * br, WP, 1,
                             tq + 64 * khalf * WQ + 32 * bc, WQ, 1, 64);
  __syncthreads();
  // the second halves of the reduction travel through LDS (the operands are spent)
  lds_f* const red = tp + blk * 1024;
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
      if (row < pw && col < qw) C[(size_t)row * n + col] = near ? old[e] - v : v;
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
      !enable_large_lds((const void*)potrf_sub_kernel<2, 2>, SUB_SMEM_BYTES) ||
      !enable_large_lds((const void*)potrf_sub_kernel<4, 1>, SUB_SMEM_BYTES))
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
    Pend = std::min(P0 + GROUP_BLOCKS, Tmax);
    auto total_items = [&](int count, auto&& items) {
      long sum = 0;
      for (int i = 0; i < count; ++i) sum += std::max(0, (int)items(Ts[i]));
      return sum;
    };
    for (int p = P0; p < Pend; ++p) {
      const int na = active(p + 1);
      // diagonal block p; beside it, panel p-1's update of the group's rows beyond p
      // (rows p+1 .. Pend-1; row p got it right after panel p-1)
      auto rest_items = [&](int T) { return (std::min(Pend, T) - p - 1) * (T - p - 1); };
      if (p == P0 || total_items(na, rest_items) == 0) {
        hipLaunchKernelGGL(potrf_diag_kernel, dim3(na), dim3(256), DIAG_SMEM_BYTES, stream,
                           table, p, info);
      } else {
        bool first = true;
        for_worklists(na, rest_items, [&](const WorkList& wl, int grid) {
          const int nd = first ? na : 0;
          first = false;
          hipLaunchKernelGGL(potrf_step_kernel, dim3(nd + grid), dim3(NTHREADS), DIAG_SMEM_BYTES,
                             stream, table, p, info, nd, p + 1, Pend, wl);
        });
      }
      const int nb = active(p + 2);
      if (nb == 0) continue;
      auto panel_items = [&](int T) { return T - p - 1; };
      if (total_items(nb, panel_items) <= SUB_MAX_TILES) {
        for_worklists(nb, [&](int T) { return 4 * std::max(0, panel_items(T)); },
                      [&](const WorkList& wl, int grid) {
                        hipLaunchKernelGGL((potrf_sub_kernel<4, 1>), dim3(grid), dim3(SUB_THREADS),
                                           SUB_SMEM_BYTES, stream, table, p, 0, 0, wl);
                      });
      } else
      for_worklists(nb, panel_items, [&](const WorkList& wl, int grid) {
        if (grid <= FINE_MAX_TILES)
          hipLaunchKernelGGL(potrf_fine_kernel, dim3(grid), dim3(FINE_THREADS), FINE_SMEM_BYTES,
                             stream, table, p, 0, 0, wl);
        else
          KFAC_LAUNCH_TILE2(potrf_panel_kernel, dim3(grid), stream, table, p, wl);
      });
      if (p + 1 < Pend) {
        // panel p's update of block row p+1 (the next diagonal block and row panel need it);
        // the group's other rows get it beside the next diagonal block
        auto row_items = [&](int T) { return T > p + 1 ? T - p - 1 : 0; };
        if (total_items(nb, row_items) <= SUB_MAX_TILES) {
          for_worklists(nb, [&](int T) { return 4 * std::max(0, row_items(T)); },
                        [&](const WorkList& wl, int grid) {
                          hipLaunchKernelGGL((potrf_sub_kernel<2, 2>), dim3(grid),
                                             dim3(SUB_THREADS), SUB_SMEM_BYTES, stream, table, p,
                                             1, p + 2, wl);
                        });
        } else
        for_worklists(nb, row_items,
                      [&](const WorkList& wl, int grid) {
                        if (grid <= FINE_MAX_TILES)
                          hipLaunchKernelGGL(potrf_fine_kernel, dim3(grid), dim3(FINE_THREADS),
                                             FINE_SMEM_BYTES, stream, table, p, 1, p + 2, wl);
                        else
                          KFAC_LAUNCH_TILE2(potrf_trail_kernel, dim3(grid), stream, table, p, 1,
                                            p + 1, p + 2, wl);
                      });
      }
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
  return run_batched(mats, MODE_INVERSE, info, ptr, STATIC_SCRATCH_BYTES, (hipStream_t)stream);
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
