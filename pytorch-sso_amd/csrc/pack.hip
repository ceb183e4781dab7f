// Wire format of the factors: symmetric matrices travel as their upper triangle,
// row by row (element (y, x), x >= y, at  n*y - y*(y+1)/2 + x), everything else as
// it lies in memory, all arrays of a list back to back in one flat buffer.
// One launch packs or unpacks a whole list.
//
//   pack     one workgroup per matrix row: A[y][y..n) -> a contiguous run of the buffer
//   unpack   one workgroup per 64x64 tile of the upper triangle: the tile is read
//            from the buffer into LDS and written twice, as it is and transposed,
//            so that both triangles of the matrix are filled with row-contiguous
//            stores
//   flat     4096-element chunks, loads ahead of stores
#include <algorithm>
#include <vector>

#include "common.h"
#include "gemm_core.h"

namespace kfac {

struct PackDesc {
  float* mat;      // the array (matrix or flat)
  float* vec;      // its place in the buffer
  long numel;      // flat arrays: element count
  int n;           // triangular: matrix size
  int tri;
};

constexpr int PACK_CHUNK = 64;
struct PackChunk {
  PackDesc d[PACK_CHUNK];
};

__global__ void pack_setup_kernel(PackChunk chunk, PackDesc* table, int offset, int count) {
  const int i = threadIdx.x;
  if (i < count) table[offset + i] = chunk.d[i];
}

constexpr int FLAT_CHUNK = 4096;
constexpr int PT = 64;     // unpack tile

__device__ __forceinline__ long tri_index(int n, int y, int x) {
  return (long)n * y - (long)y * (y + 1) / 2 + x;
}

template <bool UNPACK>
__global__ __launch_bounds__(256) void pack_kernel(const PackDesc* table, const WorkList wl) {
  __shared__ float tile[PT][PT + 1];
  int arr, local;
  work_find(wl, arr, local);
  const PackDesc d = table[arr];
  const int t = threadIdx.x;
  if (!d.tri) {
    const float* src = UNPACK ? d.vec : d.mat;
    float* dst = UNPACK ? d.mat : d.vec;
    const long base = (long)local * FLAT_CHUNK + t;
    float v[FLAT_CHUNK / 256];
#pragma unroll
    for (int k = 0; k < FLAT_CHUNK / 256; ++k) {
      const long i = base + (long)k * 256;
      v[k] = i < d.numel ? src[i] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < FLAT_CHUNK / 256; ++k) {
      const long i = base + (long)k * 256;
      if (i < d.numel) dst[i] = v[k];
    }
    return;
  }
  const int n = d.n;
  if (!UNPACK) {
    const int y = local;
    const float* src = d.mat + (size_t)y * n + y;
    float* dst = d.vec + tri_index(n, y, y);
    const int len = n - y;
    for (int x0 = t; x0 < len; x0 += 256 * 4) {
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = x0 + 256 * k < len ? src[x0 + 256 * k] : 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (x0 + 256 * k < len) dst[x0 + 256 * k] = v[k];
    }
    return;
  }
  // unpack one tile (bi <= bj) of the upper triangle
  const int T = (n + PT - 1) / PT;
  int bi, bj;
  upper_tile(local, T, bi, bj);
  for (int e = t; e < PT * PT; e += 256) {
    const int r = e / PT, c = e - r * PT;
    const int y = bi * PT + r, x = bj * PT + c;
    if (y < n && x < n && x >= y) tile[r][c] = d.vec[tri_index(n, y, x)];
  }
  __syncthreads();
  for (int e = t; e < PT * PT; e += 256) {
    const int r = e / PT, c = e - r * PT;
    const int y = bi * PT + r, x = bj * PT + c;
    if (y < n && x < n) {
      // inside a diagonal tile the part left of the diagonal comes from its mirror image
      d.mat[(size_t)y * n + x] = x >= y ? tile[r][c] : tile[c][r];
    }
  }
  if (bi != bj) {
    for (int e = t; e < PT * PT; e += 256) {
      const int r = e / PT, c = e - r * PT;       // r over x, c over y: rows of the mirrored tile
      const int x = bj * PT + r, y = bi * PT + c;
      if (y < n && x < n) d.mat[(size_t)x * n + y] = tile[c][r];
    }
  }
}

static size_t pack_workspace(int count) { return (size_t)count * sizeof(PackDesc); }

static long packed_elems(long numel, int n, int tri) {
  return tri ? (long)n * (n + 1) / 2 : numel;
}

template <bool UNPACK>
static int run_pack(int count, float* const* arrays, const int64_t* numel, const int* dims,
                    const int* triangular, float* buffer, int64_t offset, void* workspace,
                    size_t workspace_bytes, hipStream_t stream) {
  if (count == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < pack_workspace(count)) return KFAC_ERR_WORKSPACE;
  PackDesc* table = (PackDesc*)workspace;
  std::vector<int> items(count);
  long pos = offset;
  for (int s0 = 0; s0 < count; s0 += PACK_CHUNK) {
    PackChunk chunk;
    const int cnt = std::min(PACK_CHUNK, count - s0);
    for (int k = 0; k < cnt; ++k) {
      const int i = s0 + k;
      PackDesc& d = chunk.d[k];
      d.mat = arrays[i];
      d.vec = buffer + pos;
      d.numel = numel[i];
      d.n = dims[i];
      d.tri = triangular[i] ? 1 : 0;
      pos += packed_elems(numel[i], dims[i], d.tri);
      if (!d.tri)
        items[i] = (int)((numel[i] + FLAT_CHUNK - 1) / FLAT_CHUNK);
      else if (!UNPACK)
        items[i] = dims[i];
      else {
        const int T = (dims[i] + PT - 1) / PT;
        items[i] = T * (T + 1) / 2;
      }
    }
    hipLaunchKernelGGL(pack_setup_kernel, dim3(1), dim3(PACK_CHUNK), 0, stream, chunk, table, s0,
                       cnt);
  }
  for (int s0 = 0; s0 < count; s0 += WL_MAX) {
    WorkList wl;
    wl.first = s0;
    wl.n = std::min(WL_MAX, count - s0);
    wl.cum[0] = 0;
    for (int i = 0; i < wl.n; ++i) wl.cum[i + 1] = wl.cum[i] + items[s0 + i];
    for (int i = wl.n + 1; i <= WL_MAX; ++i) wl.cum[i] = wl.cum[wl.n];
    if (wl.cum[wl.n] > 0)
      hipLaunchKernelGGL(pack_kernel<UNPACK>, dim3(wl.cum[wl.n]), dim3(256), 0, stream, table, wl);
  }
  return launch_status();
}

static bool pack_args_ok(int count, const void* arrays, const int64_t* numel, const int* dims,
                         const int* triangular, const void* buffer, int64_t offset) {
  if (count < 0 || offset < 0) return false;
  if (count == 0) return true;
  if (!arrays || !numel || !dims || !triangular || !buffer) return false;
  for (int i = 0; i < count; ++i) {
    if (!((const void* const*)arrays)[i]) return false;
    if (triangular[i]) {
      if (dims[i] <= 0 || dims[i] > 16384 || numel[i] != (int64_t)dims[i] * dims[i]) return false;
    } else if (numel[i] <= 0) {
      return false;
    }
  }
  return true;
}

}  // namespace kfac

using namespace kfac;

extern "C" {

size_t kfac_pack_workspace_bytes(int count) { return count > 0 ? pack_workspace(count) : 0; }

int64_t kfac_packed_numel(int count, const int64_t* numel, const int* dims, const int* triangular) {
  if (count <= 0 || !numel || !dims || !triangular) return 0;
  int64_t total = 0;
  for (int i = 0; i < count; ++i) total += packed_elems(numel[i], dims[i], triangular[i] ? 1 : 0);
  return total;
}

int kfac_pack_batched(int count, const float* const* arrays, const int64_t* numel, const int* dims,
                      const int* triangular, float* buffer, int64_t offset, void* workspace,
                      size_t workspace_bytes, void* stream) {
  if (!pack_args_ok(count, arrays, numel, dims, triangular, buffer, offset)) return KFAC_ERR_ARG;
  return run_pack<false>(count, (float* const*)arrays, numel, dims, triangular, buffer, offset,
                         workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_unpack_batched(int count, float* const* arrays, const int64_t* numel, const int* dims,
                        const int* triangular, const float* buffer, int64_t offset,
                        void* workspace, size_t workspace_bytes, void* stream) {
  if (!pack_args_ok(count, arrays, numel, dims, triangular, buffer, offset)) return KFAC_ERR_ARG;
  return run_pack<true>(count, arrays, numel, dims, triangular, (float*)buffer, offset, workspace,
                        workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
