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
  int pad;
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

template <bool SAMPLE>
__global__ __launch_bounds__(NTHREADS) void precond_first_kernel(const LayerDesc* table,
                                                                 const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  const int item = xcd_remap(local, ta * tg);
  const int bi = item / tg, bj = item - bi * tg;   // bi over dA, bj over dG
  EpiStore epi{m.Tt, m.dG, m.dA, m.dG, 1.f, 0.f, false};
  if (SAMPLE) {
    // noise E is a plain dG x dA matrix; U_G is upper triangular: L(k, i) = U_G[i][k], k >= i
    DenseKM P{m.V, nullptr, m.dA, m.dA, 0};
    DenseMK Q{m.L, m.dG, m.dG};
    gemm_tile(P, Q, bi * BM, bj * BN, bj * BN, m.dG, false, epi, smem);
  } else {
    DenseKM P{m.V, m.vb, m.dAw, m.dA, m.vb ? 2 : 0};
    DenseKM Q{m.L, nullptr, m.dG, m.dG, 0};
    gemm_tile(P, Q, bi * BM, bj * BN, 0, m.dG, false, epi, smem);
  }
}

template <bool SAMPLE>
__global__ __launch_bounds__(NTHREADS) void precond_second_kernel(const LayerDesc* table,
                                                                 const WorkList wl) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  int layer, local;
  work_find(wl, layer, local);
  const LayerDesc m = table[layer];
  const int ta = tiles128(m.dA), tg = tiles128(m.dG);
  const int item = xcd_remap(local, ta * tg);
  const int bi = item / ta, bj = item - bi * ta;   // bi over dG, bj over dA
  DenseKM P{m.Tt, nullptr, m.dG, m.dG, 0};
  DenseKM Q{m.R, nullptr, m.dA, m.dA, 0};
  EpiSplit epi{m.outW, m.outb, m.meanW, m.meanb, m.dG, m.dA, m.dAw, m.scale};
  // U_A is upper triangular: rows a > j are zero, so the sum stops at the tile's last column
  const int kend = SAMPLE ? min(m.dA, (bj + 1) * BN) : m.dA;
  gemm_tile(P, Q, bi * BM, bj * BN, 0, kend, false, epi, smem);
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static size_t precond_workspace(int layers, const int* dG, const int* dA) {
  size_t bytes = 2 * align256((size_t)layers * sizeof(LayerDesc));     // one table per product
  for (int l = 0; l < layers; ++l) bytes += align256((size_t)dG[l] * dA[l] * sizeof(float));
  return bytes;
}

static int run_layers(int layers, const int* dG, const int* dA, const float* const* L,
                      const float* const* R, const float* const* V, const float* const* vb,
                      const float* const* meanW, const float* const* meanb, float* const* outW,
                      float* const* outb, const int* has_bias, float scale, bool sample,
                      void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (layers == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < precond_workspace(layers, dG, dA)) return KFAC_ERR_WORKSPACE;
  // Longest tiles first, so that the tail of a launch is made of short tiles: each of
  // the two products walks the layers in the order of ITS reduction length (dG for the
  // first, dA for the second), through a descriptor table of its own.
  const size_t table_bytes = align256((size_t)layers * sizeof(LayerDesc));
  LayerDesc* tables[2] = {(LayerDesc*)workspace, (LayerDesc*)((char*)workspace + table_bytes)};
  char* tbase = (char*)workspace + 2 * table_bytes;
  std::vector<size_t> toff(layers);
  size_t off = 0;
  for (int l = 0; l < layers; ++l) {
    toff[l] = off;
    off += align256((size_t)dG[l] * dA[l] * sizeof(float));
  }
  std::vector<int> order[2];
  for (int pass = 0; pass < 2; ++pass) {
    const int* key = pass == 0 ? dG : dA;
    order[pass].resize(layers);
    for (int l = 0; l < layers; ++l) order[pass][l] = l;
    std::stable_sort(order[pass].begin(), order[pass].end(),
                     [&](int a, int b) { return key[a] > key[b]; });
    for (int s0 = 0; s0 < layers; s0 += LAYER_CHUNK) {
      LayerChunk chunk;
      const int cnt = std::min(LAYER_CHUNK, layers - s0);
      for (int k = 0; k < cnt; ++k) {
        const int l = order[pass][s0 + k];
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
        d.pad = 0;
      }
      hipLaunchKernelGGL(layer_setup_kernel, dim3(1), dim3(LAYER_CHUNK), 0, stream, chunk,
                         tables[pass], s0, cnt);
    }
  }
  // both products have one tile per 128 x 128 block of the [dG, dA] result; every
  // first product is enqueued before any second one (stream order is the dependency)
  for (int pass = 0; pass < 2; ++pass) {
    LayerDesc* const table = tables[pass];
    for (int s0 = 0; s0 < layers; s0 += WL_MAX) {
      WorkList wl;
      wl.first = s0;
      wl.n = std::min(WL_MAX, layers - s0);
      wl.cum[0] = 0;
      for (int i = 0; i < wl.n; ++i) {
        const int l = order[pass][s0 + i];
        wl.cum[i + 1] = wl.cum[i] + cdiv(dG[l], BM) * cdiv(dA[l], BN);
      }
      for (int i = wl.n + 1; i <= WL_MAX; ++i) wl.cum[i] = wl.cum[wl.n];
      const dim3 grid(wl.cum[wl.n]);
      if (pass == 0) {
        if (sample) KFAC_LAUNCH_TILE2(precond_first_kernel<true>, grid, stream, table, wl);
        else KFAC_LAUNCH_TILE2(precond_first_kernel<false>, grid, stream, table, wl);
      } else {
        if (sample) KFAC_LAUNCH_TILE2(precond_second_kernel<true>, grid, stream, table, wl);
        else KFAC_LAUNCH_TILE2(precond_second_kernel<false>, grid, stream, table, wl);
      }
    }
  }
  return launch_status();
}

}  // namespace kfac

using namespace kfac;

extern "C" {

size_t kfac_precondition_workspace_bytes(int layers, const int* dG, const int* dA) {
  if (layers <= 0 || !dG || !dA) return 0;
  return precond_workspace(layers, dG, dA);
}

int kfac_precondition_batched(int layers, const int* dG, const int* dA,
                              const float* const* Ginv, const float* const* Ainv,
                              float* const* gradW, float* const* gradb, void* workspace,
                              size_t workspace_bytes, void* stream) {
  if (layers < 0 || (layers > 0 && (!dG || !dA || !Ginv || !Ainv || !gradW || !gradb)))
    return KFAC_ERR_ARG;
  std::vector<int> hb(layers);
  for (int l = 0; l < layers; ++l) {
    if (dG[l] <= 0 || dA[l] <= 0 || !Ginv[l] || !Ainv[l] || !gradW[l]) return KFAC_ERR_ARG;
    if ((int64_t)dA[l] * dA[l] > (int64_t)1 << 28 || (int64_t)dG[l] * dG[l] > (int64_t)1 << 28 ||
        (int64_t)dA[l] * dG[l] > (int64_t)1 << 28)
      return KFAC_ERR_ARG;
    hb[l] = gradb[l] != nullptr;
    if (hb[l] && dA[l] < 2) return KFAC_ERR_ARG;
  }
  return run_layers(layers, dG, dA, Ginv, Ainv, (const float* const*)gradW,
                    (const float* const*)gradb, nullptr, nullptr, gradW, gradb, hb.data(), 1.f,
                    false, workspace, workspace_bytes, (hipStream_t)stream);
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
                    hb.data(), std_scale, true, workspace, workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
