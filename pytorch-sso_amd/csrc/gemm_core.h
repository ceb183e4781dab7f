// fp32 MFMA GEMM tile engine for gfx950 (CDNA4, wave64).
//
// One workgroup of 256 threads (4 waves, 2x2) computes a 128x128 tile of
//     C[m][n] = sum_k  P(k, m) * Q(k, n)          k in [kbeg, kend)
// with v_mfma_f32_32x32x2_f32.  Each wave owns a 64x64 sub-tile (2x2 MFMA
// blocks, 64 accumulator registers).  Operands are described by functors that
// map (k, m) to a global-memory element, so the same engine serves
//   * factor builds (X^T X for Linear, implicit im2col for Conv2d),
//   * the trailing updates / triangular products of the blocked inverse,
//   * the two chained preconditioning GEMMs,
// without ever materialising a transposed, concatenated or unfolded copy.
//
// Operand functor contract (details in operands.h):
//   static constexpr int layout;      KM: consecutive m are contiguous in memory
//                                     MK: consecutive k are contiguous in memory
//   MS mstate(int m) / KS kstate(int k, bool valid): per-index precomputation
//   unsigned off(MS, KS): byte offset for a raw buffer load; an element outside
//                         the operand gets an offset beyond the buffer and reads 0
// The layout only chooses how the 256 threads sweep the 16x128 chunk so that
// global loads coalesce, and how the chunk sits in LDS:
//   KM chunk -> lds[k][m]   (row length = tile width), MFMA lanes read ds_read_b32
//   MK chunk -> lds[m][KC+4],                           MFMA lanes read ds_read_b128
// Within a 16-deep slice of a chunk the k values are consumed in the order
//   step (j,s), lane half h  ->  k = 8j + 4h + s
// for both operands, which is a permutation of the reduction index and so does
// not change the product.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>

namespace kfac {

constexpr int BM = 128;          // tile rows of the default (2x2 waves) configuration
constexpr int BN = 128;          // tile cols of the default configuration
constexpr int NTHREADS = 256;    // threads of the default configuration

// A configuration is WM x WN waves, each owning a 64x64 sub-tile:
//   tile = (64*WM) x (64*WN), threads = 64*WM*WN.
// 2x2 is the default; 1x1 (one wave, 64x64) serves small factors, where a
// 128-wide tile would be mostly padding.
// KC = 16 is the reduction depth per LDS stage (32 MFMAs per wave and stage);
// two stages of the 2x2 configuration take 40 KiB, so that three workgroups
// fit the 160 KiB of a CU.
template <int WM, int WN>
struct Cfg {
  static constexpr int TM = 64 * WM;
  static constexpr int TN = 64 * WN;
  static constexpr int NT = 64 * WM * WN;
  static constexpr int KC = 16;
  static constexpr int LDS_MK = KC + 4;          // padded row of an MK chunk (conflict-free b128)
  static constexpr int P_FLOATS = LDS_MK * TM;   // >= KC*TM and TM*LDS_MK
  static constexpr int Q_FLOATS = LDS_MK * TN;
  static constexpr int SMEM_FLOATS = 2 * (P_FLOATS + Q_FLOATS);
};
constexpr int SMEM_FLOATS = Cfg<2, 2>::SMEM_FLOATS;   // 40 KiB

enum { KM = 0, MK = 1 };

__host__ __device__ inline int tiles128(int d) { return (d + BM - 1) / BM; }

typedef float v16f __attribute__((ext_vector_type(16)));

// LDS pointers carry their address space explicitly: through a generic pointer
// the compiler emits FLAT loads/stores, whose completion is counted together
// with global loads, and the wait before the MFMAs would then also wait for the
// prefetch of the next chunk.
typedef __attribute__((address_space(3))) float lds_f;
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4f lds_f4;

// Division of an index below 2^31 by a divisor fixed per launch, as a multiply
// and a shift: with l = ceil(log2 d) and m = ceil(2^(31+l) / d) (which fits 32
// bits), floor(n / d) == (n * m) >> (31 + l) for every n < 2^31.  The operand
// functors turn a reduction index into (image, row, column) once per thread and
// chunk; a hardware-less integer division there costs about 40 instructions.
struct FastDiv {
  unsigned m, sh;
  FastDiv() = default;
  __host__ __device__ explicit FastDiv(unsigned d) {
    unsigned l = 0;
    while ((1ull << l) < d) ++l;
    sh = 31 + l;
    m = (unsigned)(((1ull << sh) + d - 1) / d);
  }
  __host__ __device__ __forceinline__ int div(int n) const {
    return (int)(((unsigned long long)(unsigned)n * m) >> sh);
  }
};

// ---- raw buffer addressing (see the operand contract in operands.h) ----------
constexpr unsigned INV_M = 0x80000000u;
constexpr unsigned INV_K = 0x40000000u;
constexpr long MAX_OPERAND_BYTES = 1L << 30;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float* p) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, (int)MAX_OPERAND_BYTES,
                                           0x00020000);
}
__device__ __forceinline__ float buffer_load(__amdgpu_buffer_rsrc_t r, unsigned off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0));
}
typedef unsigned v4u __attribute__((ext_vector_type(4)));
// four consecutive elements (dword-aligned); the range check covers the group as a whole
__device__ __forceinline__ v4f buffer_load4(__amdgpu_buffer_rsrc_t r, unsigned off) {
  return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
}

// ---------------------------------------------------------------------------
// global -> register -> LDS staging of one operand chunk (KC x ROWS elements
// swept by NT threads)
// ---------------------------------------------------------------------------
// An operand type with `static constexpr bool square = true` has its elements
// squared on the way into LDS (diagonal curvature: sums of squared gradients).
template <class T, class = void>
struct squares_elements : std::false_type {};
template <class T>
struct squares_elements<T, std::void_t<decltype(T::square)>> : std::bool_constant<T::square> {};

template <class OP, int ROWS, int NT, int KC>
struct Stager {
  static constexpr int LDS_MK = KC + 4;
  static constexpr int CNT = KC * ROWS / NT;            // elements per thread
  static constexpr int NM = (OP::layout == KM) ? 1 : CNT;
  static constexpr int KSTEP = NT / ROWS;               // KM: k rows per sweep
  static constexpr int MSTEP = NT / KC;                 // MK: m rows per sweep
  typename OP::MS ms[NM];
  float regs[CNT];
  unsigned onebits;    // element i is the constant 1 (and inside the k range)

  // (thread index within a group of NT threads: a workgroup may hold several groups,
  // each computing a tile of its own)
  __device__ __forceinline__ void init(const OP& op, int m0) {
    const int t = threadIdx.x & (NT - 1);
    if (OP::layout == KM) {
      ms[0] = op.mstate(m0 + (t % ROWS));
    } else {
#pragma unroll
      for (int i = 0; i < NM; ++i) ms[i] = op.mstate(m0 + (t / KC) + MSTEP * i);
    }
    onebits = 0;
  }

  // Issue the buffer loads of one chunk.  Elements outside the operand or the
  // k range come back as 0 from the hardware's range check; the loaded values
  // are not touched until commit, so nothing here waits on memory.
  __device__ __forceinline__ void fetch(const OP& op, int k0, int kend) {
    const int t = threadIdx.x & (NT - 1);
    const __amdgpu_buffer_rsrc_t rs = op.rsrc();
    unsigned oneb = 0;
    if (OP::layout == KM) {
#pragma unroll
      for (int i = 0; i < CNT; ++i) {
        const int k = k0 + (t / ROWS) + KSTEP * i;
        const bool kin = k < kend;
        const typename OP::KS ks = op.kstate(k, kin);
        regs[i] = buffer_load(rs, op.off(ms[0], ks));
        if constexpr (OP::has_second) {
          if (op.second()) regs[i] += buffer_load(op.rsrc2(), op.off2(ms[0], ks));
        }
        oneb |= (unsigned)(op.is_one(ms[0]) && kin) << i;
      }
    } else {
      const int k = k0 + (t % KC);
      const bool kin = k < kend;
      const typename OP::KS ks = op.kstate(k, kin);
#pragma unroll
      for (int i = 0; i < CNT; ++i) {
        regs[i] = buffer_load(rs, op.off(ms[i], ks));
        oneb |= (unsigned)(op.is_one(ms[i]) && kin) << i;
      }
    }
    onebits = oneb;
  }

  __device__ __forceinline__ void commit(lds_f* tile) const {
    const int t = threadIdx.x & (NT - 1);
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      float v = ((onebits >> i) & 1u) ? 1.f : regs[i];
      if (squares_elements<OP>::value) v *= v;
      if (OP::layout == KM)
        tile[((t / ROWS) + KSTEP * i) * ROWS + (t % ROWS)] = v;
      else
        tile[((t / KC) + MSTEP * i) * LDS_MK + (t % KC)] = v;
    }
  }
};

// An operand in the KM layout (consecutive m contiguous in memory) may offer vector access:
// `static constexpr bool vec4 = true` and `int vec_cols() const`, the number of leading
// columns that are plain memory, of which any four consecutive ones may be fetched with one
// 16-byte load.  A tile that lies inside those columns is staged by VecStager: a quarter of
// the load and LDS-store instructions of the element-wise stager (109 -> 127 TFLOP/s for a
// product of two such operands on 128-wide tiles).
template <class T, class = void>
struct offers_vec4 : std::false_type {};
template <class T>
struct offers_vec4<T, std::void_t<decltype(T::vec4)>> : std::bool_constant<T::vec4 && T::layout == KM> {};

template <class OP, int ROWS, int NT, int KC>
struct VecStager {
  static constexpr int G = ROWS / 4;             // 16-byte groups per k row
  static constexpr int KSTEP = NT / G;           // k rows per sweep
  static constexpr int CNT = KC / KSTEP;         // groups per thread
  static_assert(NT % G == 0 && KC % KSTEP == 0, "the threads sweep whole k rows");
  typename OP::MS ms;
  v4f regs[CNT];

  __device__ __forceinline__ void init(const OP& op, int m0) {
    const int t = threadIdx.x & (NT - 1);
    ms = op.mstate(m0 + 4 * (t % G));
  }
  __device__ __forceinline__ void fetch(const OP& op, int k0, int kend) {
    const int t = threadIdx.x & (NT - 1);
    const __amdgpu_buffer_rsrc_t rs = op.rsrc();
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int k = k0 + (t / G) + KSTEP * i;
      regs[i] = buffer_load4(rs, op.off(ms, op.kstate(k, k < kend)));
    }
  }
  __device__ __forceinline__ void commit(lds_f* tile) const {
    const int t = threadIdx.x & (NT - 1);
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      v4f v = regs[i];
      if (squares_elements<OP>::value) v *= v;
      *(lds_f4*)(tile + ((t / G) + KSTEP * i) * ROWS + 4 * (t % G)) = v;
    }
  }
};

template <class OP, int ROWS, int NT, int KC, bool VEC>
using StagerFor = std::conditional_t<VEC && offers_vec4<OP>::value, VecStager<OP, ROWS, NT, KC>,
                                     Stager<OP, ROWS, NT, KC>>;

// the tile [m0, m0 + rows) of the operand can go through VecStager (true for operands
// that have no vector access: they are staged as ever)
template <class OP>
__device__ __forceinline__ bool vec_tile_ok(const OP& op, int m0, int rows) {
  if constexpr (offers_vec4<OP>::value) return m0 + rows <= op.vec_cols();
  return true;
}

// fragments of one operand for the 8 MFMA steps of a 16-deep slice starting at
// k = kofs of the staged chunk: f[sub][4j+s]
template <int LAYOUT, int ROWS, int LDS_MK>
__device__ __forceinline__ void load_frags(const lds_f* tile, int base, int r, int h, int kofs,
                                           float (&f)[2][8]) {
  if (LAYOUT == KM) {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int s = 0; s < 4; ++s)
          f[sub][4 * j + s] = tile[(kofs + 8 * j + 4 * h + s) * ROWS + base + 32 * sub + r];
  } else {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const v4f v = *(const lds_f4*)(&tile[(base + 32 * sub + r) * LDS_MK + kofs + 8 * j + 4 * h]);
        f[sub][4 * j + 0] = v.x;
        f[sub][4 * j + 1] = v.y;
        f[sub][4 * j + 2] = v.z;
        f[sub][4 * j + 3] = v.w;
      }
  }
}

// ---------------------------------------------------------------------------
// The tile engine.  `same` = P and Q describe the same columns (diagonal tile
// of a symmetric product): Q is then neither fetched nor stored.
// EPI::store(row, col, value) receives every element of the tile (global
// coordinates row = m0 + ..., col = n0 + ...).
// ---------------------------------------------------------------------------
// An epilogue with `static constexpr bool indexed = true` receives the running
// index (a*2 + b)*16 + i of each accumulator instead of its position in C.
template <class T, class = void>
struct indexed_epilogue : std::false_type {};
template <class T>
struct indexed_epilogue<T, std::void_t<decltype(T::indexed)>> : std::bool_constant<T::indexed> {};

// An epilogue with `static constexpr bool reads_output = true` offers
// reads() / fetch(row, col) / store_with(row, col, v, old) next to store().
template <class T, class = void>
struct reading_epilogue : std::false_type {};
template <class T>
struct reading_epilogue<T, std::void_t<decltype(T::reads_output)>>
    : std::bool_constant<T::reads_output> {};

// Position in C of accumulator element i of block (a, b) of the calling thread;
// the epilogue visits (a, b, i) in lexicographic order, 64 elements per thread.
template <int WM, int WN>
__device__ __forceinline__ void acc_coords(int m0, int n0, int a, int b, int i, int& row,
                                           int& col) {
  const int lane = threadIdx.x & 63;
  const int wave = (threadIdx.x & (64 * WM * WN - 1)) >> 6;
  const int r = lane & 31, h = lane >> 5;
  row = m0 + (wave / WN) * 64 + 32 * a + 8 * (i >> 2) + 4 * h + (i & 3);
  col = n0 + (wave % WN) * 64 + 32 * b + r;
}

// The MFMAs of k-steps [S0, S1) of a 16-deep slice.  A diagonal tile of a symmetric product
// is symmetric itself: with SKIP its 32x32 blocks below the diagonal are not computed, and
// the blocks above it are stored twice.  The 10 blocks of a 128-wide tile are dealt 3, 2, 2, 3
// over its four waves: the waves on the diagonal quadrants take the three blocks of theirs,
// and the quadrant above the diagonal is shared by the wave that owns it (upper two blocks)
// and the wave of the quadrant below the diagonal (lower two), so the tile is done in three
// quarters of the time.  The single wave of a 64-wide tile takes its three blocks.  The
// matrix cores this leaves alone serve the other workgroups of the compute unit; a launch
// with few workgroups per unit has little to gain and pays for the mirrored stores.
enum { WAVE_FULL = 0, WAVE_DIAG = 1, WAVE_ROW0 = 2, WAVE_ROW1 = 3 };
template <int S0, int S1, bool SKIP>
__device__ __forceinline__ void mma_slice(const float (&fa)[2][8], const float (&fb)[2][8],
                                          v16f (&acc)[2][2], int mode) {
  if (!SKIP || mode == WAVE_FULL) {
#pragma unroll
    for (int s = S0; s < S1; ++s)
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a][s], fb[b][s], acc[a][b], 0, 0, 0);
  } else if (mode == WAVE_DIAG) {
#pragma unroll
    for (int s = S0; s < S1; ++s) {
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][s], fb[0][s], acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][s], fb[1][s], acc[0][1], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][s], fb[1][s], acc[1][1], 0, 0, 0);
    }
  } else if (mode == WAVE_ROW0) {
#pragma unroll
    for (int s = S0; s < S1; ++s) {
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][s], fb[0][s], acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][s], fb[1][s], acc[0][1], 0, 0, 0);
    }
  } else {
#pragma unroll
    for (int s = S0; s < S1; ++s) {
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][s], fb[0][s], acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][s], fb[1][s], acc[1][1], 0, 0, 0);
    }
  }
}

// acc_coords for a wave whose quadrant starts at (wm, wn) of the tile
__device__ __forceinline__ void quad_coords(int m0, int n0, int wm, int wn, int a, int b, int i,
                                            int& row, int& col) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  row = m0 + wm + 32 * a + 8 * (i >> 2) + 4 * h + (i & 3);
  col = n0 + wn + 32 * b + r;
}

// The reduction loop of a tile: stages 16-deep chunks of both operands through LDS (double
// buffered) and accumulates into the calling wave's four blocks.  VEC: operands that offer
// vector access are staged with 16-byte loads (the caller has checked that the tile allows it).
template <int WM, int WN, bool SAME, bool SKIP, bool VEC, class OPP, class OPQ>
__device__ __forceinline__ void gemm_tile_loop(const OPP& P, const OPQ& Q, int m0, int n0, int kbeg,
                                               int kend, float* smem, int wm, int wn, int mode,
                                               v16f (&acc)[2][2]) {
  typedef Cfg<WM, WN> C;
  constexpr bool same = SAME;
  const int t = threadIdx.x & (C::NT - 1);
  const int lane = t & 63;
  const int r = lane & 31;
  const int h = lane >> 5;
  constexpr int KC = C::KC;
  StagerFor<OPP, C::TM, C::NT, C::KC, VEC> sp;
  StagerFor<OPQ, C::TN, C::NT, C::KC, VEC> sq;
  sp.init(P, m0);
  if (!same) sq.init(Q, n0);

  lds_f* const sm = (lds_f*)smem;
  constexpr int STAGE = C::P_FLOATS + C::Q_FLOATS;

  const int nchunks = (kend - kbeg + KC - 1) / KC;
  if (nchunks > 0) {
    sp.fetch(P, kbeg, kend);
    if (!same) sq.fetch(Q, kbeg, kend);
    sp.commit(sm);
    if (!same) sq.commit(sm + C::P_FLOATS);
  }
  __syncthreads();

  for (int c = 0; c < nchunks; ++c) {
    const int cur = c & 1;
    const bool more = (c + 1) < nchunks;
    if (more) {
      sp.fetch(P, kbeg + (c + 1) * KC, kend);
      if (!same) sq.fetch(Q, kbeg + (c + 1) * KC, kend);
    }
    const lds_f* const tpc = sm + cur * STAGE;
    const lds_f* const tqc = tpc + C::P_FLOATS;
    lds_f* const tpn = sm + (cur ^ 1) * STAGE;
    // The chunk is consumed in 16-deep slices.  The LDS writes of the NEXT chunk
    // are issued before the last slice, so that they (and the wait for the
    // global loads that feed them) sit in the shadow of MFMAs instead of in
    // front of the barrier.
#pragma unroll
    for (int sl = 0; sl < KC / 16; ++sl) {
      float fa[2][8], fb[2][8];
      {
        load_frags<OPP::layout, C::TM, C::LDS_MK>(tpc, wm, r, h, 16 * sl, fa);
        if (same)
          load_frags<OPP::layout, C::TM, C::LDS_MK>(tpc, wn, r, h, 16 * sl, fb);
        else
          load_frags<OPQ::layout, C::TN, C::LDS_MK>(tqc, wn, r, h, 16 * sl, fb);
      }
      if (sl == KC / 16 - 1) {
        mma_slice<0, 4, SKIP>(fa, fb, acc, mode);
        if (more) {
          sp.commit(tpn);
          if (!same) sq.commit(tpn + C::P_FLOATS);
        }
        mma_slice<4, 8, SKIP>(fa, fb, acc, mode);
      } else {
        mma_slice<0, 8, SKIP>(fa, fb, acc, mode);
      }
    }
    __syncthreads();
  }

}

template <int WM, int WN, bool SAME, bool SKIP, class OPP, class OPQ, class EPI>
__device__ __forceinline__ void gemm_tile_impl(const OPP& P, const OPQ& Q, int m0, int n0,
                                               int kbeg, int kend, EPI& epi, float* smem) {
  typedef Cfg<WM, WN> C;
  constexpr bool same = SAME;
  const int t = threadIdx.x & (C::NT - 1);
  const int lane = t & 63;
  const int wave = t >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  int wm = (wave / WN) * 64;
  int wn = (wave % WN) * 64;
  static_assert(SAME || !SKIP, "only a diagonal tile of a symmetric product has blocks to skip");
  static_assert(!SKIP || (WM == WN && WM <= 2), "skipping is written for 64- and 128-wide tiles");
  int mode = WAVE_FULL;
  if (SKIP) {
    if (wm == wn) {
      mode = WAVE_DIAG;
    } else if (wm < wn) {
      mode = WAVE_ROW0;
    } else {             // the quadrant below the diagonal: the lower half of the one above
      mode = WAVE_ROW1;
      wm = 0;
      wn = 64;
    }
  }

  v16f acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  // (uniform per workgroup: the tile lies inside the columns that vector loads may fetch)
  constexpr bool can_vec = offers_vec4<OPP>::value || (!SAME && offers_vec4<OPQ>::value);
  bool vec = false;
  if constexpr (can_vec) vec = vec_tile_ok(P, m0, C::TM) && (same || vec_tile_ok(Q, n0, C::TN));
  if constexpr (can_vec) {
    if (vec)
      gemm_tile_loop<WM, WN, SAME, SKIP, true>(P, Q, m0, n0, kbeg, kend, smem, wm, wn, mode, acc);
  }
  if (!vec)
    gemm_tile_loop<WM, WN, SAME, SKIP, false>(P, Q, m0, n0, kbeg, kend, smem, wm, wn, mode, acc);

  // A diagonal tile of a symmetric product: the blocks above the tile's diagonal are
  // stored at their mirror position too, the blocks below it were not computed.
  auto computed = [&](int a, int b) {
    return !SKIP || (mode == WAVE_DIAG ? a <= b : a == (mode == WAVE_ROW0 ? 0 : 1));
  };
  auto mirrored = [&](int a, int b) { return SKIP && computed(a, b) && (wm + 32 * a < wn + 32 * b); };

  if constexpr (reading_epilogue<EPI>::value) {
    // C = alpha*acc + beta*C_old: the old values are loaded 32 at a time ahead of the
    // stores.  Interleaved load/store pairs would each wait for their own load (a store
    // to C may alias the next load of C, so the compiler keeps them in order).
    if (epi.reads()) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        float old[32];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int row, col;
            quad_coords(m0, n0, wm, wn, a, b, i, row, col);
            old[b * 16 + i] = computed(a, b) ? epi.fetch(row, col) : 0.f;
          }
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int row, col;
            quad_coords(m0, n0, wm, wn, a, b, i, row, col);
            if (computed(a, b)) epi.store_with(row, col, acc[a][b][i], old[b * 16 + i]);
            // (the old values are symmetric like the new ones)
            if (mirrored(a, b)) epi.store_with(col, row, acc[a][b][i], old[b * 16 + i]);
          }
      }
      return;
    }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        int row, col;
        quad_coords(m0, n0, wm, wn, a, b, i, row, col);
        if constexpr (indexed_epilogue<EPI>::value) {
          static_assert(!SKIP, "indexed epilogues do not take skipped blocks");
          epi.store_at((a * 2 + b) * 16 + i, acc[a][b][i]);     // index known at compile time
        } else {
          if (computed(a, b)) epi.store(row, col, acc[a][b][i]);
          if (mirrored(a, b)) epi.store(col, row, acc[a][b][i]);
        }
      }
}

// SKIP_LOWER: a diagonal tile (`same`) leaves out its blocks below the diagonal.
template <int WM, int WN, bool SKIP_LOWER = false, class OPP, class OPQ, class EPI>
__device__ __forceinline__ void gemm_tile_cfg(const OPP& P, const OPQ& Q, int m0, int n0,
                                              int kbeg, int kend, bool same, EPI& epi,
                                              float* smem) {
  if constexpr (std::is_same<OPP, OPQ>::value) {
    if (same) {
      gemm_tile_impl<WM, WN, true, SKIP_LOWER && !indexed_epilogue<EPI>::value>(
          P, Q, m0, n0, kbeg, kend, epi, smem);
      return;
    }
  }
  gemm_tile_impl<WM, WN, false, false>(P, Q, m0, n0, kbeg, kend, epi, smem);
}

// default configuration: 128x128 tile, 256 threads
template <class OPP, class OPQ, class EPI>
__device__ __forceinline__ void gemm_tile(const OPP& P, const OPQ& Q, int m0, int n0, int kbeg,
                                          int kend, bool same, EPI& epi, float* smem) {
  gemm_tile_cfg<2, 2>(P, Q, m0, n0, kbeg, kend, same, epi, smem);
}

// ---------------------------------------------------------------------------
// A tile whose reduction was cut into `nparts` pieces, each computed by a workgroup of its
// own that stored its raw 128x128 partial (EpiPartial) at parts + piece * 128 * 128: a
// workgroup of a LATER launch adds the pieces up in order and hands every element to the
// epilogue.  (Finishing in the same launch, by the piece that arrives last, was measured:
// the device-wide fences it needs write back and invalidate the whole L2 of an XCD each
// time, and the operand panels that the other workgroups share through that L2 with them.)
// ---------------------------------------------------------------------------
// pieces of a reduction of `blocks` 128-blocks cut at `pb` blocks (pb <= 0: not cut)
__host__ __device__ inline int piece_count(int blocks, int pb) {
  return pb > 0 ? (blocks + pb - 1) / pb : 1;
}

// (`stride`: floats from one piece of the tile to the next)
template <class EPI>
__device__ __forceinline__ void splitk_sum(const float* parts, int nparts, int m0, int n0,
                                           const EPI& epi, size_t stride = BM * BN) {
  constexpr int TILE = BM * BN;
  constexpr int PER_THREAD = TILE / 4 / NTHREADS;      // float4 groups per thread: 16
  // piece by piece, the 16 loads of a thread in flight together
  v4f acc[PER_THREAD];
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i)
    acc[i] = *reinterpret_cast<const v4f*>(parts + 4 * ((int)threadIdx.x + NTHREADS * i));
  for (int q = 1; q < nparts; ++q) {
    const float* p = parts + (size_t)q * stride;
    v4f v[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i)
      v[i] = *reinterpret_cast<const v4f*>(p + 4 * ((int)threadIdx.x + NTHREADS * i));
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) acc[i] += v[i];
  }
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int e = 4 * ((int)threadIdx.x + NTHREADS * i);
    const int row = m0 + (e >> 7), col = n0 + (e & (BN - 1));
    epi.store(row, col, acc[i].x);
    epi.store(row, col + 1, acc[i].y);
    epi.store(row, col + 2, acc[i].z);
    epi.store(row, col + 3, acc[i].w);
  }
}

// Workgroups are handed to the 8 XCDs round-robin in dispatch order, and each
// XCD has its own L2.  This maps the dispatch index `id` of a 1-D problem of
// `total` work items so that every XCD walks a CONTIGUOUS range of items:
// neighbouring tiles, which share operand panels, then hit the same L2.
__device__ __forceinline__ int xcd_remap(int id, int total) {
  const int x = id & 7, q = total >> 3, r = total & 7;
  const int base = x < r ? x * (q + 1) : r * (q + 1) + (x - r) * q;
  return base + (id >> 3);
}

// Workgroups go to the 8 XCDs round-robin by dispatch index g.  The n items of one
// product occupy the dispatch indices [c0, c0 + n); this permutation of [0, n) gives
// every XCD a contiguous run of them.
__device__ __forceinline__ int xcd_remap_range(int g, int c0, int n) {
  const int s = c0 & 7;
  const int v = g - c0 + s;        // index in a virtual range that starts at a multiple of 8
  const int x = v & 7;
  const int tv = n + s;
  int base = 0;
#pragma unroll
  for (int y = 0; y < 8; ++y) {
    const int cnt = ((tv - y + 7) >> 3) - (y < s ? 1 : 0);
    base += y < x ? cnt : 0;
  }
  return base + (v >> 3) - (x < s ? 1 : 0);
}


// Batched launches (one for many matrices or layers of different sizes) use a 1-D
// grid of exactly the workgroups needed: cum[i] is the first work item of the i-th
// listed matrix (table index first + i), cum[n] the grid size.  (A rectangular grid
// "largest tile count x matrices" would start tens of thousands of workgroups
// that only find out that their matrix is too small.)
constexpr int WL_MAX = 128;
struct WorkList {
  int n, first;
  int cum[WL_MAX + 1];
};

// matrix (table index) and local work item of work item `item` of the list
__device__ __forceinline__ void work_find_item(const WorkList& wl, int item, int& mat,
                                               int& local) {
  int lo = 0, hi = wl.n;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (wl.cum[mid] <= item) lo = mid; else hi = mid;
  }
  mat = wl.first + lo;
  local = item - wl.cum[lo];
}

// ... of the calling workgroup, in a launch whose grid is the list
__device__ __forceinline__ void work_find(const WorkList& wl, int& mat, int& local) {
  work_find_item(wl, (int)blockIdx.x, mat, local);
}

// tile index t (0-based, row-major over the upper triangle incl. diagonal of a
// T x T block grid) -> (bi, bj), bi <= bj
__device__ __forceinline__ void upper_tile(int t, int T, int& bi, int& bj) {
  int i = 0;
  int rowlen = T;
  // closed form guess then fix-up (T is at most a few hundred)
  const float fT = 2.f * T + 1.f;
  i = (int)((fT - sqrtf(fT * fT - 8.f * (float)t)) * 0.5f);
  if (i < 0) i = 0;
  if (i > T - 1) i = T - 1;
  // start(i) = i*T - i*(i-1)/2
  while (i > 0 && (i * T - (i * (i - 1)) / 2) > t) --i;
  while (i + 1 < T && ((i + 1) * T - ((i + 1) * i) / 2) <= t) ++i;
  (void)rowlen;
  bi = i;
  bj = i + (t - (i * T - (i * (i - 1)) / 2));
}

}  // namespace kfac
