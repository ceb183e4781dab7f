// Preconditioning  U = G^-1 [dW | db] A^-1  and posterior sampling
// P = [mW | mb] + s * U_G E U_A  for a whole set of layers in two launches.
//
// Both are two chained products on the MFMA tile engine with the intermediate
// kept transposed so that every operand is read along its contiguous dimension:
//   T^T[a][i] = sum_k V[k][a] * L[k][i]      (V = [dW|db] or E, L = G^-1 or U_G^T)
//   U[i][j]   = sum_a T^T[a][i] * R[a][j]    (R = A^-1 or U_A)
// [dW | db] is never concatenated: the bias column is read from its own vector,
// and the result is written straight back into the two gradient tensors.
#include <algorithm>
#include <vector>

#include "common.h"
#include "operands.h"

namespace kfac {

struct LayerDesc {
  const float* L;        // dG x dG : G^-1 (symmetric) or U_G (upper, sampling)
  const float* R;        // dA x dA : A^-1 or U_A
  const float* V;        // dG x dAw: weight gradient, or noise (dG x dA) when sampling
  const float* vb;       // dG      : bias gradient (nullptr: none, or noise carries it)
  const float* meanW;    // sampling: mean of the weight, else nullptr
  const float* meanb;
  float* outW;           // dG x dAw
  float* outb;           // dG or nullptr
  float* Tt;             // dA x dG scratch
  int dG, dA, dAw;       // dAw = dA - (has bias)
  float scale;
  int flags;         // factored preconditioning: bit 0 L is Wg, bit 1 R is Wa (else the inverses)
  float* parts;      // pieces of the tiles whose reduction is cut (see tile_item)
};

constexpr int LAYER_CHUNK = 32;
struct LayerChunk {
  LayerDesc d[LAYER_CHUNK];
};

__global__ void layer_setup_kernel(LayerChunk chunk, LayerDesc* table, int offset, int count) {
  const int i = threadIdx.x;
  if (i < count) table[offset + i] = chunk.d[i];
}

// result tile -> the weight tensor and the bias vector, optionally mean + scale * acc
struct EpiSplit {
  float* W;
  float* b;
  const float* mW;
  const float* mb;
  int dG, dA, dAw;
  float scale;
  static constexpr bool reads_output = true;     // the means, when sampling
  __device__ __forceinline__ bool reads() const { return mW != nullptr; }
  __device__ __forceinline__ float fetch(int row, int col) const {
    if (row < dG && col < dA) {
      if (col < dAw) return mW[(size_t)row * dAw + col];
      return mb ? mb[row] : 0.f;
    }
    return 0.f;
  }
  __device__ __forceinline__ void store_with(int row, int col, float v, float old) const {
    if (row < dG && col < dA) {
      if (col < dAw)
        W[(size_t)row * dAw + col] = old + scale * v;
      else
        b[row] = old + scale * v;
    }
  }
  __device__ __forceinline__ void store(int row, int col, float v) const {
    if (row < dG && col < dA) {
      if (col < dAw) {
        const size_t idx = (size_t)row * dAw + col;
        W[idx] = (mW ? mW[idx] : 0.f) + scale * v;
      } else {
        b[row] = (mb ? mb[row] : 0.f) + scale * v;
      }
    }
  }
};

// ---------------------------------------------------------------------------
// The products.  Explicit inverses:  U = G^-1 V A^-1, two products:
//   first    T^T[a][i] = sum_k V[k][a] G^-1[k][i]            (T = G^-1 V, kept transposed)
//   second   U[i][j]   = sum_a T^T[a][i] A^-1[a][j]
// An inverse may instead be given by its triangular factor Y (upper, Y Y^T = inverse: the
// inverse of the Cholesky factor, which the batched inversion delivers where the explicit
// inverse is not asked for; it then skips the n^3/3 product Y Y^T of that matrix).  Bit 0 of
// a layer's `flags` says that L is Yg, bit 1 that R is Ya.  A factored side takes two
// products with the triangular operand, each over the non-zero part of its reduction only
// (half of a dense product), in place of the one dense product:
//   first    T^T[a][i] = sum_{k <= i} V[k][a] Yg[k][i]       (T = Yg^T V)
//   second   X[i][j]   = sum_{a <= j} T^T[a][i] Ya[a][j]     (X = T Ya)
//   third    X'[i][j]  = sum_{a >= j} X[i][a] Ya[j][a]       (X' = X Ya^T)   layers with Ya
//   fourth   U[i][j]   = sum_{k >= i} Yg[i][k] X'[k][j]      (U = Yg X')     layers with Yg
// so that the first two read their operand exactly as they read an explicit inverse, only
// over a shorter range.  The last product a layer takes part in writes the gradients; the
// results in between live in the two halves of the layer's scratch (T^T in the first; the
// result of the second and third product in whichever half that product does not read).
//
// The reduction of a tile against a triangular operand runs from or to the tile's own
// position along one tile index (`fast` below), so its length varies from one block to all
// of them.  Such a layer's tiles are dispatched longest first: all tiles of the longest
// reduction, then the next shorter, so that the launch ends on its shortest tiles.
// Workgroups go to the 8 XCDs in turn by dispatch index; consecutive tiles share the
// triangular operand's panel and an XCD keeps meeting the same few panels of the other
// operand, so no remapping is needed for the L2s.  Dense layers keep the contiguous-range
// mapping.  Posterior sampling (U_G E U_A, both upper triangular) uses the first two
// products with its own operand layouts.
// ---------------------------------------------------------------------------

// A reduction against a triangular operand of T blocks is up to T blocks long, and a launch
// lasts at least as long as its longest tile: a 4608-deep tile is 150 MFLOP on ONE compute
// unit.  Where that is longer than the launch would take if its work were spread evenly
// (few layers, or few tiles: the driver decides per product), the reductions are cut into
// pieces of at most `pb` blocks, each a work item of the same launch that stores a raw
// partial tile; a second, short launch adds the pieces of every cut tile up in order and
// applies the epilogue (precond_finish_kernel).  Piece j exists for the tiles whose
// reduction is longer than j * pb blocks: tfast - j * pb values of `fast`.  pb == 0: no
// reduction is cut.
// work items of a layer in one product: tiles x pieces
__host__ __device__ inline int piece_items(int tslow, int tfast, bool tri, int pb) {
  if (pb <= 0) return tslow * tfast;
  if (!tri) return tslow * tfast * piece_count(tfast, pb);    // dense: all reductions tfast blocks
  int n = 0;
  for (int j = 0; j * pb < tfast; ++j) n += tslow * (tfast - j * pb);
  return n;
}

// (slow, fast) tile indices of work item `local` of a layer with tslow x tfast tiles.
// `tri`: the reduction length depends on `fast`; it grows with it if `grows`.
struct TileItem {
  int slow, fast;
  int piece, pieces;     // which piece of the tile's reduction, of how many
};
__device__ __forceinline__ TileItem tile_item(int local, int tslow, int tfast, bool tri,
                                              bool grows, int pb) {
  TileItem it;
  it.piece = 0;
  it.pieces = 1;
  if (tri) {
    // piece j of all tiles that have one, then piece j + 1; within a piece the longest
    // reductions first
    int j = 0;
    if (pb > 0)
      while (local >= tslow * (tfast - j * pb)) {
        local -= tslow * (tfast - j * pb);
        ++j;
      }
    const int rank = local / tslow;
    it.slow = local - rank * tslow;
    it.fast = grows ? tfast - 1 - rank : rank;
    it.piece = j;
    it.pieces = piece_count(grows ? it.fast + 1 : tfast - it.fast, pb);
  } else {
    // a dense operand: every reduction is tfast blocks long; piece after piece
    const int tiles = tslow * tfast;
    it.pieces = piece_count(tfast, pb);
    it.piece = local / tiles;
    const int item = xcd_remap(local - it.piece * tiles, tiles);
    it.slow = item / tfast;
    it.fast = item - it.slow * tfast;
  }
  return it;
}

// One tile of a product: the whole reduction [k0, k1) into `epi`, or one piece of it as a
// raw partial into the layer's piece area (tile `tile_id`, room for `max_pieces` each).
template <class OPP, class OPQ, class EPI>
__device__ __forceinline__ void tile_or_piece(const LayerDesc& m, const TileItem& it, int tile_id,
                                              int max_pieces, int pb, const OPP& P, const OPQ& Q,
                                              int m0, int n0, int M, int N, int k0, int k1,
                                              const EPI& epi, float* smem) {
  if (it.pieces == 1) {
    EPI e = epi;
    gemm_tile(P, Q, m0, n0, k0, k1, false, e, smem);
    return;
  }
  const int kbeg = k0 + it.piece * (pb * BM);
  const int kend = min(k1, kbeg + pb * BM);
  float* parts = m.parts + ((size_t)tile_id * max_pieces + it.piece) * (BM * BN);
  EpiPartial part{parts, m0, n0, M, N, BN};
  gemm_tile(P, Q, m0, n0, kbeg, kend, false, part, smem);
}

// where the products of a layer between the first and the last put their result
__device__ __forceinline__ float* second_half(const LayerDesc& m) {
  return m.Tt + (size_t)m.dG * m.dA;
}

// where the second, third and fourth product of a layer put their result
__device__ __forceinline__ EpiSplit second_epilogue(const LayerDesc& m) {
  return m.flags == 0 ? EpiSplit{m.outW, m.outb, nullptr, nullptr, m.dG, m.dA, m.dAw, 1.f}
                      : EpiSplit{second_half(m), nullptr, nullptr, nullptr, m.dG, m.dA, m.dA, 1.f};
}
__device__ __forceinline__ EpiSplit sample_epilogue(const LayerDesc& m) {
  return EpiSplit{m.outW, m.outb, m.meanW, m.meanb, m.dG, m.dA, m.dAw, m.scale};
}
__device__ __forceinline__ EpiSplit third_epilogue(const LayerDesc& m) {
  return (m.flags & 1) ? EpiSplit{m.Tt, nullptr, nullptr, nullptr, m.dG, m.dA, m.dA, 1.f}
                       : EpiSplit{m.outW, m.outb, nullptr, nullptr, m.dG, m.dA, m.dAw, 1.f};
}
__device__ __forceinline__ EpiSplit fourth_epilogue(const LayerDesc& m) {
  return EpiSplit{m.outW, m.outb, nullptr, nullptr, m.dG, m.dA, m.dAw, 1.f};
}

template <bool SAMPLE>
__global__ __launch_bounds__(NTHREADS, 3) void precond_first_kernel(const LayerDesc* table,
                                                                 const WorkList wl, int pb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  EpiStore epi{m.Tt, m.dG, m.dA, m.dG, 1.f, 0.f, false};
  if (SAMPLE) {
    // noise E is a plain dG x dA matrix; U_G is upper triangular: L(k, i) = U_G[i][k], k >= i
    const TileItem it = tile_item(local, ta, tg, true, false, pb);
    const int bi = it.slow, bj = it.fast;            // bi over dA, bj over dG
    DenseKM P{m.V, nullptr, m.dA, m.dA, 0};
    DenseMK Q{m.L, m.dG, m.dG};
    tile_or_piece(m, it, bi + ta * bj, piece_count(tg, pb), pb, P, Q, bi * BM, bj * BN, m.dA, m.dG,
                  bj * BN, m.dG, epi, smem);
  } else {
    const bool tri = m.flags & 1;
    const TileItem it = tile_item(local, ta, tg, tri, true, pb);
    const int bi = it.slow, bj = it.fast;            // bi over dA, bj over dG
    DenseKM P{m.V, m.vb, m.dAw, m.dA, m.vb ? 2 : 0};
    DenseKM Q{m.L, nullptr, m.dG, m.dG, 0};
    tile_or_piece(m, it, bi + ta * bj, piece_count(tg, pb), pb, P, Q, bi * BM, bj * BN, m.dA, m.dG,
                  0, tri ? min(m.dG, (bj + 1) * BN) : m.dG, epi, smem);
  }
}

template <bool SAMPLE>
__global__ __launch_bounds__(NTHREADS, 3) void precond_second_kernel(const LayerDesc* table,
                                                                 const WorkList wl, int pb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  DenseKM P{m.Tt, nullptr, m.dG, m.dG, 0};
  DenseKM Q{m.R, nullptr, m.dA, m.dA, 0};
  if (SAMPLE) {
    // U_A is upper triangular: rows a > j are zero, so the sum stops at the tile's last column
    const TileItem it = tile_item(local, tg, ta, true, true, pb);
    const int bi = it.slow, bj = it.fast;            // bi over dG, bj over dA
    tile_or_piece(m, it, bi + tg * bj, piece_count(ta, pb), pb, P, Q, bi * BM, bj * BN, m.dG, m.dA,
                  0, min(m.dA, (bj + 1) * BN), sample_epilogue(m), smem);
  } else {
    const bool tri = m.flags & 2;
    const TileItem it = tile_item(local, tg, ta, tri, true, pb);
    const int bi = it.slow, bj = it.fast;            // bi over dG, bj over dA
    tile_or_piece(m, it, bi + tg * bj, piece_count(ta, pb), pb, P, Q, bi * BM, bj * BN, m.dG, m.dA,
                  0, tri ? min(m.dA, (bj + 1) * BN) : m.dA, second_epilogue(m), smem);
  }
}

// third product, layers whose R is the factor Ya:  X' = X Ya^T, reduction a >= j
__global__ __launch_bounds__(NTHREADS, 3) void precond_third_kernel(const LayerDesc* table,
                                                                const WorkList wl, int pb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  const TileItem it = tile_item(local, tg, ta, true, false, pb);
  const int bi = it.slow, bj = it.fast;              // bi over dG, bj over dA
  DenseMK P{second_half(m), m.dA, m.dG};
  DenseMK Q{m.R, m.dA, m.dA};
  tile_or_piece(m, it, bi + tg * bj, piece_count(ta, pb), pb, P, Q, bi * BM, bj * BN, m.dG, m.dA,
                bj * BN, m.dA, third_epilogue(m), smem);
}

// fourth product, layers whose L is the factor Yg:  U = Yg X', reduction k >= i
__global__ __launch_bounds__(NTHREADS, 3) void precond_fourth_kernel(const LayerDesc* table,
                                                                 const WorkList wl, int pb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  const TileItem it = tile_item(local, ta, tg, true, false, pb);
  const int bi = it.fast, bj = it.slow;              // bi over dG, bj over dA
  DenseMK P{m.L, m.dG, m.dG};
  DenseKM Q{(m.flags & 2) ? m.Tt : second_half(m), nullptr, m.dA, m.dA, 0};
  tile_or_piece(m, it, bj + ta * bi, piece_count(tg, pb), pb, P, Q, bi * BM, bj * BN, m.dG, m.dA,
                bi * BM, m.dG, fourth_epilogue(m), smem);
}

// The tiles of product `product` (0..3) whose reduction was cut: pieces added up in order,
// result through the product's epilogue.  One work item per tile of the layers that take
// part with a triangular operand; a tile of one piece was finished by its product.
__global__ __launch_bounds__(NTHREADS) void precond_finish_kernel(const LayerDesc* table,
                                                                  const WorkList wl, int product,
                                                                  int pb, int sample) {
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  // (slow, fast) as the product numbers them; `local` = slow + tslow * fast = the tile id
  const bool over_g = product == 0 || product == 3;      // the reduction runs over dG
  const int tslow = over_g ? ta : tg, tfast = over_g ? tg : ta;
  const int fast = local / tslow, slow = local - fast * tslow;
  const bool grows = sample ? product == 1 : product < 2;
  const bool tri = sample || (m.flags & (over_g ? 1 : 2));
  const int pieces = piece_count(!tri ? tfast : (grows ? fast + 1 : tfast - fast), pb);
  if (pieces == 1) return;
  const float* parts = m.parts + (size_t)local * piece_count(tfast, pb) * (BM * BN);
  // rows of the result: dA for the first product (T^T), dG for the others
  int bi, bj;
  if (product == 0) { bi = slow; bj = fast; }          // bi over dA, bj over dG
  else if (product == 3) { bi = fast; bj = slow; }     // bi over dG, bj over dA
  else { bi = slow; bj = fast; }                       // bi over dG, bj over dA
  if (product == 0)
    splitk_sum(parts, pieces, bi * BM, bj * BN, EpiStore{m.Tt, m.dG, m.dA, m.dG, 1.f, 0.f, false});
  else if (product == 1)
    splitk_sum(parts, pieces, bi * BM, bj * BN, sample ? sample_epilogue(m) : second_epilogue(m));
  else if (product == 2)
    splitk_sum(parts, pieces, bi * BM, bj * BN, third_epilogue(m));
  else
    splitk_sum(parts, pieces, bi * BM, bj * BN, fourth_epilogue(m));
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

constexpr int PRODUCTS = 4;

// Piece size of each product from the shape of its launch.  flags == nullptr: every side of
// every layer is a triangular factor (what the scratch is sized for).
static void plan_pieces(int layers, const int* dG, const int* dA, const int* flags, bool any_tri,
                        int (&pbs)[4], bool sample = false) {
  for (int product = 0; product < 4; ++product) {
    long work = 0;
    int longest = 0;
    const bool over_g = product == 0 || product == 3;
    for (int l = 0; any_tri && !(sample && product >= 2) && l < layers; ++l) {
      const int ta = cdiv(dA[l], BN), tg = cdiv(dG[l], BM);
      const int f = flags ? flags[l] : 3;
      const int tslow = over_g ? ta : tg, tfast = over_g ? tg : ta;
      const bool tri = over_g ? (f & 1) : (f & 2);
      if (product >= 2 && !tri) continue;
      work += tri ? (long)tslow * tfast * (tfast + 1) / 2 : (long)tslow * tfast * tfast;
      longest = std::max(longest, tfast);
    }
    pbs[product] = any_tri ? piece_blocks(work, longest) : 0;
  }
}

// floats of the piece area of a layer under the piece sizes `pbs`: room for the pieces of
// the longest reduction, for every tile
static size_t piece_floats(int dG, int dA, const int (&pbs)[4]) {
  const int ta = cdiv(dA, BN), tg = cdiv(dG, BM);
  int most = 1;
  for (int product = 0; product < 4; ++product) {
    const bool over_g = product == 0 || product == 3;
    most = std::max(most, piece_count(over_g ? tg : ta, pbs[product]));
  }
  return most > 1 ? (size_t)ta * tg * most * (BM * BN) : 0;
}

// scratch: one descriptor table per product, then per layer dG*dA floats (twice that when
// `factored`: a layer with a factored side keeps two results in flight) and its piece area
static size_t precond_workspace(int layers, const int* dG, const int* dA, bool factored) {
  size_t bytes = PRODUCTS * align256((size_t)layers * sizeof(LayerDesc));
  // (the piece area is there for both queries: posterior sampling, which shares the query of
  // the explicit preconditioning, multiplies by triangular factors as well)
  int pbs[4];
  plan_pieces(layers, dG, dA, nullptr, true, pbs);
  for (int l = 0; l < layers; ++l) {
    bytes += align256((size_t)(factored ? 2 : 1) * dG[l] * dA[l] * sizeof(float));
    bytes += align256(piece_floats(dG[l], dA[l], pbs) * sizeof(float));
  }
  return bytes;
}

// flags: per layer, bit 0 L is the factor Yg, bit 1 R is the factor Ya (nullptr: none)
static int run_layers(int layers, const int* dG, const int* dA, const float* const* L,
                      const float* const* R, const float* const* V, const float* const* vb,
                      const float* const* meanW, const float* const* meanb, float* const* outW,
                      float* const* outb, const int* has_bias, float scale, bool sample,
                      const int* flags, void* workspace, size_t workspace_bytes,
                      hipStream_t stream) {
  if (layers == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < precond_workspace(layers, dG, dA, flags != nullptr))
    return KFAC_ERR_WORKSPACE;
  bool any[PRODUCTS] = {true, true, false, false};
  for (int l = 0; flags && l < layers; ++l) {
    any[2] |= (flags[l] & 2) != 0;
    any[3] |= (flags[l] & 1) != 0;
  }
  // Longest tiles first, so that the tail of a launch is made of short tiles: each
  // product walks the layers in the order of ITS reduction length (dG for the first and
  // fourth, dA for the second and third), through a descriptor table of its own.
  const size_t table_bytes = align256((size_t)layers * sizeof(LayerDesc));
  char* tbase = (char*)workspace + PRODUCTS * table_bytes;
  // pieces as large as the scratch was sized for, at least (the query assumed that every
  // side is a triangular factor), and none where it left no room
  const std::vector<int> no_flags(layers, 0);     // explicit inverses on both sides
  int pbs_room[4], pbs[PRODUCTS];
  const int* const real_flags = flags ? flags : (sample ? nullptr : no_flags.data());
  plan_pieces(layers, dG, dA, nullptr, true, pbs_room);
  plan_pieces(layers, dG, dA, real_flags, true, pbs, sample);
  for (int product = 0; product < PRODUCTS; ++product)
    pbs[product] = pbs[product] > 0 && pbs_room[product] > 0
                       ? std::max(pbs[product], pbs_room[product]) : 0;
  std::vector<size_t> toff(layers), poff(layers);
  size_t off = 0;
  for (int l = 0; l < layers; ++l) {
    toff[l] = off;
    off += align256((size_t)(flags ? 2 : 1) * dG[l] * dA[l] * sizeof(float));
    poff[l] = off;
    off += align256(piece_floats(dG[l], dA[l], pbs_room) * sizeof(float));
  }
  // per product: is the reduction of layer l against a triangular operand, over how many
  // blocks (tfast), with how many tiles across (tslow)
  auto shape = [&](int product, int l, bool& takes_part, bool& tri, int& tslow, int& tfast) {
    const int ta = cdiv(dA[l], BN), tg = cdiv(dG[l], BM);
    const bool gfac = sample || (flags && (flags[l] & 1)), afac = sample || (flags && (flags[l] & 2));
    const bool over_g = product == 0 || product == 3;
    tslow = over_g ? ta : tg;
    tfast = over_g ? tg : ta;
    tri = over_g ? gfac : afac;
    takes_part = product < 2 || (tri && !sample);
  };
  // work items of layer l in a product: its tiles x pieces, or none where it takes no part
  auto items = [&](int product, int l) {
    bool part, tri;
    int tslow, tfast;
    shape(product, l, part, tri, tslow, tfast);
    return part ? piece_items(tslow, tfast, tri, pbs[product]) : 0;
  };
  // ... and in the launch that finishes the cut tiles of the product
  auto finish_items = [&](int product, int l) {
    bool part, tri;
    int tslow, tfast;
    shape(product, l, part, tri, tslow, tfast);
    return part && piece_count(tfast, pbs[product]) > 1 ? tslow * tfast : 0;
  };
  std::vector<int> order(layers);
  for (int product = 0; product < PRODUCTS; ++product) {
    if (!any[product]) continue;
    LayerDesc* const table = (LayerDesc*)((char*)workspace + product * table_bytes);
    const int* key = (product == 0 || product == 3) ? dG : dA;
    for (int l = 0; l < layers; ++l) order[l] = l;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return key[a] > key[b]; });
    for (int s0 = 0; s0 < layers; s0 += LAYER_CHUNK) {
      LayerChunk chunk;
      const int cnt = std::min(LAYER_CHUNK, layers - s0);
      for (int k = 0; k < cnt; ++k) {
        const int l = order[s0 + k];
        LayerDesc& d = chunk.d[k];
        d.L = L[l];
        d.R = R[l];
        d.V = V[l];
        d.vb = vb ? vb[l] : nullptr;
        d.meanW = meanW ? meanW[l] : nullptr;
        d.meanb = meanb ? meanb[l] : nullptr;
        d.outW = outW[l];
        d.outb = outb ? outb[l] : nullptr;
        d.Tt = (float*)(tbase + toff[l]);
        d.dG = dG[l];
        d.dA = dA[l];
        d.dAw = dA[l] - (has_bias[l] ? 1 : 0);
        d.scale = scale;
        d.flags = flags ? flags[l] : 0;
        d.parts = (float*)(tbase + poff[l]);
      }
      hipLaunchKernelGGL(layer_setup_kernel, dim3(1), dim3(LAYER_CHUNK), 0, stream, chunk,
                         table, s0, cnt);
    }
    // every launch of a product is enqueued before any of the next one (stream order is
    // the dependency)
    const int pb = pbs[product];
    for (int s0 = 0; s0 < layers; s0 += WL_MAX) {
      WorkList wl;
      wl.first = s0;
      wl.n = std::min(WL_MAX, layers - s0);
      wl.cum[0] = 0;
      for (int i = 0; i < wl.n; ++i) wl.cum[i + 1] = wl.cum[i] + items(product, order[s0 + i]);
      for (int i = wl.n + 1; i <= WL_MAX; ++i) wl.cum[i] = wl.cum[wl.n];
      if (wl.cum[wl.n] == 0) continue;
      const dim3 grid(wl.cum[wl.n]);
      if (product == 0) {
        if (sample) KFAC_LAUNCH_TILE2(precond_first_kernel<true>, grid, stream, table, wl, pb);
        else KFAC_LAUNCH_TILE2(precond_first_kernel<false>, grid, stream, table, wl, pb);
      } else if (product == 1) {
        if (sample) KFAC_LAUNCH_TILE2(precond_second_kernel<true>, grid, stream, table, wl, pb);
        else KFAC_LAUNCH_TILE2(precond_second_kernel<false>, grid, stream, table, wl, pb);
      } else if (product == 2) {
        KFAC_LAUNCH_TILE2(precond_third_kernel, grid, stream, table, wl, pb);
      } else {
        KFAC_LAUNCH_TILE2(precond_fourth_kernel, grid, stream, table, wl, pb);
      }
    }
    if (pb > 0)
      for (int s0 = 0; s0 < layers; s0 += WL_MAX) {
        WorkList wl;
        wl.first = s0;
        wl.n = std::min(WL_MAX, layers - s0);
        wl.cum[0] = 0;
        for (int i = 0; i < wl.n; ++i)
          wl.cum[i + 1] = wl.cum[i] + finish_items(product, order[s0 + i]);
        for (int i = wl.n + 1; i <= WL_MAX; ++i) wl.cum[i] = wl.cum[wl.n];
        if (wl.cum[wl.n] == 0) continue;
        hipLaunchKernelGGL(precond_finish_kernel, dim3(wl.cum[wl.n]), dim3(NTHREADS), 0, stream,
                           table, wl, product, pb, sample ? 1 : 0);
      }
  }
  return launch_status();
}

}  // namespace kfac

using namespace kfac;

extern "C" {

double kfac_precondition_executed_flops(int layers, const int* dG, const int* dA,
                                        const int* g_factored, const int* a_factored) {
  if (layers <= 0 || !dG || !dA) return 0.;
  double blocks = 0.;      // 128-deep steps of 128 x 128 tiles
  for (int l = 0; l < layers; ++l) {
    const double ta = cdiv(dA[l], BN), tg = cdiv(dG[l], BM);
    const bool gfac = g_factored && g_factored[l], afac = a_factored && a_factored[l];
    // a dense operand: every tile reduces over all blocks of that side; a triangular one:
    // over 1..t blocks, twice (the factor and its transpose)
    blocks += gfac ? 2 * ta * tg * (tg + 1) / 2 : ta * tg * tg;
    blocks += afac ? 2 * tg * ta * (ta + 1) / 2 : tg * ta * ta;
  }
  return blocks * 2. * BM * BN * 128.;
}

size_t kfac_precondition_workspace_bytes(int layers, const int* dG, const int* dA) {
  if (layers <= 0 || !dG || !dA) return 0;
  return precond_workspace(layers, dG, dA, false);
}

static int check_layers(int layers, const int* dG, const int* dA, const float* const* Gop,
                        const float* const* Aop, float* const* gradW, float* const* gradb,
                        std::vector<int>& has_bias) {
  if (layers < 0 || (layers > 0 && (!dG || !dA || !Gop || !Aop || !gradW || !gradb)))
    return KFAC_ERR_ARG;
  has_bias.resize(layers);
  for (int l = 0; l < layers; ++l) {
    if (dG[l] <= 0 || dA[l] <= 0 || !Gop[l] || !Aop[l] || !gradW[l]) return KFAC_ERR_ARG;
    if ((int64_t)dA[l] * dA[l] > (int64_t)1 << 28 || (int64_t)dG[l] * dG[l] > (int64_t)1 << 28 ||
        (int64_t)dA[l] * dG[l] > (int64_t)1 << 28)
      return KFAC_ERR_ARG;
    has_bias[l] = gradb[l] != nullptr;
    if (has_bias[l] && dA[l] < 2) return KFAC_ERR_ARG;
  }
  return KFAC_OK;
}

int kfac_precondition_batched(int layers, const int* dG, const int* dA,
                              const float* const* Ginv, const float* const* Ainv,
                              float* const* gradW, float* const* gradb, void* workspace,
                              size_t workspace_bytes, void* stream) {
  std::vector<int> hb;
  const int st = check_layers(layers, dG, dA, Ginv, Ainv, gradW, gradb, hb);
  if (st != KFAC_OK) return st;
  return run_layers(layers, dG, dA, Ginv, Ainv, (const float* const*)gradW,
                    (const float* const*)gradb, nullptr, nullptr, gradW, gradb, hb.data(), 1.f,
                    false, nullptr, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t kfac_precondition_factored_workspace_bytes(int layers, const int* dG, const int* dA) {
  if (layers <= 0 || !dG || !dA) return 0;
  return precond_workspace(layers, dG, dA, true);
}

int kfac_precondition_factored_batched(int layers, const int* dG, const int* dA,
                                       const float* const* Gop, const float* const* Aop,
                                       const int* g_factored, const int* a_factored,
                                       float* const* gradW, float* const* gradb, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  std::vector<int> hb;
  const int st = check_layers(layers, dG, dA, Gop, Aop, gradW, gradb, hb);
  if (st != KFAC_OK) return st;
  std::vector<int> flags(layers);
  for (int l = 0; l < layers; ++l)
    flags[l] = ((!g_factored || g_factored[l]) ? 1 : 0) | ((!a_factored || a_factored[l]) ? 2 : 0);
  return run_layers(layers, dG, dA, Gop, Aop, (const float* const*)gradW,
                    (const float* const*)gradb, nullptr, nullptr, gradW, gradb, hb.data(), 1.f,
                    false, flags.data(), workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_sample_batched(int layers, const int* dG, const int* dA, const float* const* U_G,
                        const float* const* U_A, const float* const* noise,
                        const float* const* meanW, const float* const* meanb,
                        float* const* paramW, float* const* paramb, float std_scale,
                        void* workspace, size_t workspace_bytes, void* stream) {
  if (layers < 0 ||
      (layers > 0 && (!dG || !dA || !U_G || !U_A || !noise || !meanW || !meanb || !paramW || !paramb)))
    return KFAC_ERR_ARG;
  std::vector<int> hb(layers);
  for (int l = 0; l < layers; ++l) {
    if (dG[l] <= 0 || dA[l] <= 0 || !U_G[l] || !U_A[l] || !noise[l] || !meanW[l] || !paramW[l])
      return KFAC_ERR_ARG;
    if ((int64_t)dA[l] * dA[l] > (int64_t)1 << 28 || (int64_t)dG[l] * dG[l] > (int64_t)1 << 28 ||
        (int64_t)dA[l] * dG[l] > (int64_t)1 << 28)
      return KFAC_ERR_ARG;
    hb[l] = paramb[l] != nullptr;
    if (hb[l] && (!meanb[l] || dA[l] < 2)) return KFAC_ERR_ARG;
  }
  return run_layers(layers, dG, dA, U_G, U_A, noise, nullptr, meanW, meanb, paramW, paramb,
                    hb.data(), std_scale, true, nullptr, workspace, workspace_bytes,
                    (hipStream_t)stream);
}

}  // extern "C"
