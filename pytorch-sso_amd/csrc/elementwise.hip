// HBM-bound tails of the K-FAC step, each one launch over a whole list of
// tensors: running average / accumulation, diagonal (BatchNorm) curvature,
// diagonal inverse and preconditioning, and the fused parameter update.
#include <limits.h>

#include <algorithm>
#include <vector>

#include "common.h"

namespace kfac {

struct VecDesc {
  float* a;
  float* b;
  float* c;
  long numel;
  float s0, s1, s2, s3;
};

constexpr int VEC_CHUNK = 64;
struct VecChunk {
  VecDesc d[VEC_CHUNK];
};

__global__ void vec_setup_kernel(VecChunk chunk, VecDesc* table, int offset, int count) {
  const int i = threadIdx.x;
  if (i < count) table[offset + i] = chunk.d[i];
}

enum { OP_AXPBY = 0, OP_DIAG_INV = 1, OP_MUL = 2, OP_SGD = 3, OP_SQRT = 4, OP_MAX = 5, OP_ADDCMUL = 6 };

constexpr int EW_THREADS = 256;
constexpr int EW_PER_THREAD = 4;
constexpr int EW_BLOCK = EW_THREADS * EW_PER_THREAD;

// Each thread handles EW_PER_THREAD elements: all loads first, then the
// arithmetic, then all stores.  (Load/store pairs issued one element at a time
// would each wait for their own load: a store may alias the next load, so the
// compiler keeps them in order.)
template <int OP>
__global__ __launch_bounds__(EW_THREADS) void vec_kernel(const VecDesc* table) {
  const VecDesc m = table[blockIdx.y];
  const long nblocks = (m.numel + EW_BLOCK - 1) / EW_BLOCK;
  constexpr bool USES_B = OP == OP_AXPBY || OP == OP_MUL || OP == OP_SGD || OP == OP_MAX ||
                          OP == OP_ADDCMUL;
  constexpr bool USES_C = OP == OP_SGD || OP == OP_ADDCMUL;
  for (long blk = blockIdx.x; blk < nblocks; blk += gridDim.x) {
    const long base = blk * EW_BLOCK + threadIdx.x;
    float a[EW_PER_THREAD], b[EW_PER_THREAD], c[EW_PER_THREAD];
#pragma unroll
    for (int k = 0; k < EW_PER_THREAD; ++k) {
      const long i = base + (long)k * EW_THREADS;
      const bool in = i < m.numel;
      a[k] = in ? m.a[i] : 0.f;
      b[k] = 0.f;
      c[k] = 0.f;
      if (USES_B && in && !(OP == OP_AXPBY && m.s1 == 0.f)) b[k] = m.b[i];
      if (USES_C && in && !(OP == OP_SGD && m.s1 == 0.f)) c[k] = m.c[i];
    }
#pragma unroll
    for (int k = 0; k < EW_PER_THREAD; ++k) {
      const long i = base + (long)k * EW_THREADS;
      if (i >= m.numel) continue;
      if (OP == OP_AXPBY) {
        // b = s0 * a + s1 * b     (s1 == 0: b is not read)
        float v = m.s0 * a[k];
        if (m.s1 != 0.f) v += m.s1 * b[k];
        m.b[i] = v;
      } else if (OP == OP_DIAG_INV) {
        // b = 1 / ((s1 ? sqrt(a) : a) + s0)
        float v = a[k];
        if (m.s1 != 0.f) v = sqrtf(v);
        m.b[i] = 1.f / (v + m.s0);
      } else if (OP == OP_MUL) {
        m.b[i] = b[k] * a[k];                       // b *= a
      } else if (OP == OP_SQRT) {
        m.b[i] = sqrtf(a[k]);
      } else if (OP == OP_MAX) {
        m.b[i] = fmaxf(a[k], b[k]);
      } else if (OP == OP_ADDCMUL) {
        // b = a + s0 * b * c     (a = mean, b = noise in / parameter out, c = std)
        m.b[i] = fmaf(m.s0 * b[k], c[k], a[k]);
      } else {
        // a = param, b = grad, c = momentum buffer; s0 = lr, s1 = momentum, s2 = weight decay
        float g = b[k];
        const float p = a[k];
        if (m.s2 != 0.f) g += m.s2 * p;
        if (m.s1 != 0.f) {
          g = m.s1 * c[k] + g;
          m.c[i] = g;
        }
        m.b[i] = g;
        m.a[i] = p - m.s0 * g;
      }
    }
  }
}

// y = s0*x + s1*y on float4 (all pointers 16-byte aligned, numel % 4 == 0): the
// running average of the factors moves the most bytes of all tails.  Four float4
// per thread and iteration, loads ahead of stores.
__global__ __launch_bounds__(EW_THREADS) void axpby4_kernel(const VecDesc* table) {
  const VecDesc m = table[blockIdx.y];
  const long n4 = m.numel >> 2;
  const float4* x = reinterpret_cast<const float4*>(m.a);
  float4* y = reinterpret_cast<float4*>(m.b);
  const long stride = (long)gridDim.x * EW_THREADS;
  const bool rd = m.s1 != 0.f;
  for (long i0 = (long)blockIdx.x * EW_THREADS + threadIdx.x; i0 < n4; i0 += 4 * stride) {
    float4 a[4], b[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const long i = i0 + k * stride;
      a[k] = i < n4 ? x[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      b[k] = (rd && i < n4) ? y[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const long i = i0 + k * stride;
      if (i < n4) {
        float4 o;
        o.x = m.s0 * a[k].x + m.s1 * b[k].x;
        o.y = m.s0 * a[k].y + m.s1 * b[k].y;
        o.z = m.s0 * a[k].z + m.s1 * b[k].z;
        o.w = m.s0 * a[k].w + m.s1 * b[k].w;
        y[i] = o;
      }
    }
  }
}

// The fused update on float4 (all pointers 16-byte aligned, numel % 4 == 0): a = param,
// b = grad, c = momentum buffer; s0 = lr, s1 = momentum, s2 = weight decay.  Two float4
// of each tensor per thread and iteration, loads ahead of stores.
__device__ __forceinline__ float sgd_one(float p, float g, float c, const VecDesc& m, float& buf) {
  if (m.s2 != 0.f) g += m.s2 * p;
  if (m.s1 != 0.f) {
    g = m.s1 * c + g;
    buf = g;
  }
  return g;
}

__global__ __launch_bounds__(EW_THREADS) void sgd4_kernel(const VecDesc* table) {
  const VecDesc m = table[blockIdx.y];
  const long n4 = m.numel >> 2;
  float4* pa = reinterpret_cast<float4*>(m.a);
  float4* pb = reinterpret_cast<float4*>(m.b);
  float4* pc = reinterpret_cast<float4*>(m.c);
  const long stride = (long)gridDim.x * EW_THREADS;
  const bool mom = m.s1 != 0.f;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  for (long i0 = (long)blockIdx.x * EW_THREADS + threadIdx.x; i0 < n4; i0 += 2 * stride) {
    float4 a[2], b[2], c[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const long i = i0 + k * stride;
      const bool in = i < n4;
      a[k] = in ? pa[i] : zero;
      b[k] = in ? pb[i] : zero;
      c[k] = (in && mom) ? pc[i] : zero;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const long i = i0 + k * stride;
      if (i >= n4) continue;
      float4 g, buf = c[k];
      g.x = sgd_one(a[k].x, b[k].x, c[k].x, m, buf.x);
      g.y = sgd_one(a[k].y, b[k].y, c[k].y, m, buf.y);
      g.z = sgd_one(a[k].z, b[k].z, c[k].z, m, buf.z);
      g.w = sgd_one(a[k].w, b[k].w, c[k].w, m, buf.w);
      if (mom) pc[i] = buf;
      pb[i] = g;
      pa[i] = make_float4(a[k].x - m.s0 * g.x, a[k].y - m.s0 * g.y, a[k].z - m.s0 * g.z,
                          a[k].w - m.s0 * g.w);
    }
  }
}

static size_t vec_workspace(int count) { return (size_t)count * sizeof(VecDesc); }

static long upload_table(const std::vector<VecDesc>& descs, VecDesc* table, long per_block,
                         hipStream_t stream);

// the running average: float4 kernel for the tensors that allow it, scalar for the rest
static int run_axpby(std::vector<VecDesc>& descs, void* workspace, size_t workspace_bytes,
                     hipStream_t stream) {
  const int count = (int)descs.size();
  if (count == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < vec_workspace(count)) return KFAC_ERR_WORKSPACE;
  std::vector<VecDesc> v4, sc;
  for (const VecDesc& d : descs) {
    const bool aligned = (((uintptr_t)d.a | (uintptr_t)d.b) & 15) == 0 && (d.numel & 3) == 0;
    (aligned ? v4 : sc).push_back(d);
  }
  VecDesc* table = (VecDesc*)workspace;
  if (!v4.empty()) {
    const long maxblocks = upload_table(v4, table, 4L * EW_THREADS * 4, stream);
    long gx = std::max<long>(64, 8192 / (long)v4.size());
    gx = std::min(gx, maxblocks);
    hipLaunchKernelGGL(axpby4_kernel, dim3((unsigned)gx, (unsigned)v4.size()), dim3(EW_THREADS), 0,
                       stream, table);
  }
  if (!sc.empty()) {
    VecDesc* t2 = table + v4.size();
    const long maxblocks = upload_table(sc, t2, EW_BLOCK, stream);
    long gx = std::max<long>(64, 4096 / (long)sc.size());
    gx = std::min(gx, maxblocks);
    hipLaunchKernelGGL((vec_kernel<OP_AXPBY>), dim3((unsigned)gx, (unsigned)sc.size()),
                       dim3(EW_THREADS), 0, stream, t2);
  }
  return launch_status();
}

// copies the descriptors to the device table; returns the block count of the largest tensor
static long upload_table(const std::vector<VecDesc>& descs, VecDesc* table, long per_block,
                         hipStream_t stream) {
  const int count = (int)descs.size();
  long maxblocks = 1;
  for (int s0 = 0; s0 < count; s0 += VEC_CHUNK) {
    VecChunk chunk;
    const int cnt = std::min(VEC_CHUNK, count - s0);
    for (int k = 0; k < cnt; ++k) {
      chunk.d[k] = descs[s0 + k];
      maxblocks = std::max(maxblocks, (descs[s0 + k].numel + per_block - 1) / per_block);
    }
    hipLaunchKernelGGL(vec_setup_kernel, dim3(1), dim3(VEC_CHUNK), 0, stream, chunk, table, s0,
                       cnt);
  }
  return maxblocks;
}

template <int OP>
static int run_vec(std::vector<VecDesc>& descs, void* workspace, size_t workspace_bytes,
                   hipStream_t stream) {
  const int count = (int)descs.size();
  if (count == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < vec_workspace(count)) return KFAC_ERR_WORKSPACE;
  VecDesc* table = (VecDesc*)workspace;
  long maxblocks = 1;
  for (int s0 = 0; s0 < count; s0 += VEC_CHUNK) {
    VecChunk chunk;
    const int cnt = std::min(VEC_CHUNK, count - s0);
    for (int k = 0; k < cnt; ++k) {
      chunk.d[k] = descs[s0 + k];
      maxblocks = std::max(maxblocks, (descs[s0 + k].numel + EW_BLOCK - 1) / EW_BLOCK);
    }
    hipLaunchKernelGGL(vec_setup_kernel, dim3(1), dim3(VEC_CHUNK), 0, stream, chunk, table, s0,
                       cnt);
  }
  long gx = std::max<long>(64, 4096 / count);
  gx = std::min(gx, maxblocks);
  hipLaunchKernelGGL((vec_kernel<OP>), dim3((unsigned)gx, count), dim3(EW_THREADS), 0, stream,
                     table);
  return launch_status();
}

// ---- BatchNorm diagonal curvature ----------------------------------------

// out[row] = sum_i ((x[row][i] - shift[c]) / scale[c])^2, row = (n, c), c = row % C.
// One wave per row when rows are short (a 256-thread workgroup then covers 4
// rows), one workgroup per row otherwise; lanes stride the row so that loads
// coalesce.
template <int ROWS_PER_BLOCK>
__global__ __launch_bounds__(256) void rowsq_kernel(const float* x, const float* scale,
                                                    const float* shift, long rows, int C, int len,
                                                    float* out) {
  constexpr int TPR = 256 / ROWS_PER_BLOCK;       // threads per row
  __shared__ float red[256];
  const int sub = threadIdx.x / TPR;
  const int lane = threadIdx.x - sub * TPR;
  const long row = (long)blockIdx.x * ROWS_PER_BLOCK + sub;
  float s = 0.f;
  if (row < rows) {
    const int c = (int)(row % C);
    const float sh = shift ? shift[c] : 0.f;
    const float rs = scale ? 1.f / scale[c] : 1.f;
    const float* p = x + row * (long)len;
    int i = lane;
    if (ROWS_PER_BLOCK == 1 && (len & 3) == 0 && ((uintptr_t)x & 15) == 0) {
      // long aligned rows: float4 loads, 4 of them in flight per thread
      const float4* p4 = reinterpret_cast<const float4*>(p);
      const int len4 = len >> 2;
      for (int i4 = lane; i4 < len4; i4 += 4 * TPR) {
        float4 v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
          v[k] = i4 + k * TPR < len4 ? p4[i4 + k * TPR] : make_float4(sh, sh, sh, sh);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float a = (v[k].x - sh) * rs, b = (v[k].y - sh) * rs;
          const float c2 = (v[k].z - sh) * rs, d = (v[k].w - sh) * rs;
          s += a * a + b * b + c2 * c2 + d * d;
        }
      }
      i = len;
    }
    for (; i + 3 * TPR < len; i += 4 * TPR) {       // 4 loads in flight per thread
      const float v0 = (p[i] - sh) * rs, v1 = (p[i + TPR] - sh) * rs;
      const float v2 = (p[i + 2 * TPR] - sh) * rs, v3 = (p[i + 3 * TPR] - sh) * rs;
      s += v0 * v0 + v1 * v1 + v2 * v2 + v3 * v3;
    }
    for (; i < len; i += TPR) {
      const float v = (p[i] - sh) * rs;
      s += v * v;
    }
  }
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = TPR / 2; w > 0; w >>= 1) {
    if (lane < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (lane == 0 && row < rows) out[row] = red[threadIdx.x];
}

// out[r][i] = x[r][i] * (use_sqrt ? sqrt(w[r]) : w[r]),  rows of length len
__global__ __launch_bounds__(256) void scale_rows_kernel(const float* x, const float* w, long rows,
                                                         long len, int use_sqrt, float* out) {
  const long total = rows * len;
  const long stride = (long)gridDim.x * 256;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const float s = w[i / len];
    out[i] = x[i] * (use_sqrt ? sqrtf(s) : s);
  }
}

// w_curv[c] = alpha * sum_n sx[n][c] * sg[n][c] ; b_curv[c] = alpha * sum_n sg[n][c]
// 64 channels x 4 slices of n per workgroup: the loads of a thread are independent,
// and the four slice sums are added in slice order.
__global__ __launch_bounds__(256) void bn_combine_kernel(const float* sx, const float* sg, int N,
                                                         int C, float alpha, float* w_curv,
                                                         float* b_curv) {
  __shared__ float rw[4][64], rb[4][64];
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  float sw = 0.f, sb = 0.f;
  if (c < C) {
#pragma unroll 4
    for (int n = slice; n < N; n += 4) {
      const float g = sg[(long)n * C + c];
      sw += sx[(long)n * C + c] * g;
      sb += g;
    }
  }
  rw[slice][lane] = sw;
  rb[slice][lane] = sb;
  __syncthreads();
  if (slice == 0 && c < C) {
    w_curv[c] = alpha * (((rw[0][lane] + rw[1][lane]) + rw[2][lane]) + rw[3][lane]);
    if (b_curv) b_curv[c] = alpha * (((rb[0][lane] + rb[1][lane]) + rb[2][lane]) + rb[3][lane]);
  }
}

// Short rows (len up to 1024): one workgroup takes one channel c and all N samples,
// i.e. the rows x + (n*C + c)*len.  A wave has 8 or 16 loads (float4 where the rows
// allow it) in flight: UNROLL rows of CHUNKS loads each.  The 8 partial sums of a lane are
// folded with 10 shuffles (halving the number of values a lane carries at each of the
// first three steps).  COMBINE = false writes the row sums out[n*C + c]; COMBINE = true
// keeps them in LDS and finishes the BatchNorm curvature of the channel,
//   w_curv[c] = alpha * sum_n sx[n][c] * rowsum[n],  b_curv[c] = alpha * sum_n rowsum[n],
// summed over n in order, so that neither the row sums nor a second launch touch memory.
// These launches are short and run from a cold instruction cache: the code is kept small
// (no per-row index arithmetic, few shuffles).
constexpr int BN_MAX_ROWS = 2048;      // samples per workgroup

// The sums over n of one channel, from its row sums in LDS (all threads of the workgroup
// call this; `prod`: BN_MAX_ROWS floats of LDS)
__device__ __forceinline__ void bn_finish_channel(const float* rowsum, float* prod,
                                                  const float* sx, int N, int C, int c,
                                                  float alpha, float* w_curv, float* b_curv) {
  __syncthreads();
  // sx[n][c] * rowsum[n] by all threads, then one thread adds over n in order
  for (int q = threadIdx.x; q < N; q += 256) prod[q] = sx[(long)q * C + c] * rowsum[q];
  __syncthreads();
  if (threadIdx.x == 0) {
    float sw = 0.f, sb = 0.f;
#pragma unroll 8
    for (int n = 0; n < N; ++n) {
      sw += prod[n];
      sb += rowsum[n];
    }
    w_curv[c] = alpha * sw;
    if (b_curv) b_curv[c] = alpha * sb;
  }
}

// (channel c; `rowsum`, `prod`: BN_MAX_ROWS floats of LDS each, used with COMBINE)
template <int CHUNKS, bool VEC, bool COMBINE>
__device__ __forceinline__ void bn_rows_body(const float* x, const float* scale,
                                             const float* shift, int N, int C, int len,
                                             const float* sx, float alpha, float* out,
                                             float* w_curv, float* b_curv, int c, float* rowsum,
                                             float* prod) {
  constexpr int UNROLL = CHUNKS == 4 ? 4 : 8;      // rows in flight per wave
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int units = VEC ? len >> 2 : len;          // loads per row
  const float sh = shift ? shift[c] : 0.f;
  const float rs = scale ? 1.f / scale[c] : 1.f;
  const long stride = (long)C * len;               // from sample to sample
  const float* base = x + (long)c * len;
  for (int q0 = wave * UNROLL; q0 < N; q0 += 4 * UNROLL) {
    // every load is issued unconditionally, at an index clamped into the row (and the row
    // into the samples), so that nothing separates the loads; what a clamped load brought
    // is dropped when the squares are summed
    float4 v[UNROLL][CHUNKS];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const float* p = base + (long)min(q0 + u, N - 1) * stride;
#pragma unroll
      for (int k = 0; k < CHUNKS; ++k) {
        const int i = min(lane + 64 * k, units - 1);
        if (VEC)
          v[u][k] = reinterpret_cast<const float4*>(p)[i];
        else
          v[u][k].x = p[i];
      }
    }
    float s[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) s[u] = 0.f;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int k = 0; k < CHUNKS; ++k) {
        const float a = (v[u][k].x - sh) * rs;
        float t = a * a;
        if (VEC) {
          const float b = (v[u][k].y - sh) * rs, c2 = (v[u][k].z - sh) * rs;
          const float d = (v[u][k].w - sh) * rs;
          t += b * b + c2 * c2 + d * d;
        }
        s[u] += (lane + 64 * k < units && q0 + u < N) ? t : 0.f;
      }
    }
    // fold: after the steps with masks 32, 16, 8 a lane carries one value, that of row
    // 4*bit5 + 2*bit4 + bit3 of its lane number; masks 4, 2, 1 finish the sum
#pragma unroll
    for (int half = 4, m = 32; half >= 1; half >>= 1, m >>= 1) {
      const bool up = lane & m;
#pragma unroll
      for (int j = 0; j < half; ++j) {
        const float send = up ? s[j] : s[j + half];
        const float keep = up ? s[j + half] : s[j];
        s[j] = keep + __shfl_xor(send, m);
      }
    }
    float r = s[0];
#pragma unroll
    for (int m = 4; m > 0; m >>= 1) r += __shfl_xor(r, m);
    const int q = q0 + ((lane >> 5) & 1) * 4 + ((lane >> 4) & 1) * 2 + ((lane >> 3) & 1);
    if ((lane & 7) == 0 && q < q0 + UNROLL && q < N) {
      if (COMBINE)
        rowsum[q] = r;
      else
        out[(long)q * C + c] = r;
    }
  }
  if (COMBINE) bn_finish_channel(rowsum, prod, sx, N, C, c, alpha, w_curv, b_curv);
}

template <int CHUNKS, bool VEC, bool COMBINE>
__global__ __launch_bounds__(256) void bn_rows_kernel(const float* x, const float* scale,
                                                      const float* shift, int N, int C, int len,
                                                      const float* sx, float alpha, float* out,
                                                      float* w_curv, float* b_curv) {
  __shared__ float rowsum[COMBINE ? BN_MAX_ROWS : 1];
  __shared__ float prod[COMBINE ? BN_MAX_ROWS : 1];
  bn_rows_body<CHUNKS, VEC, COMBINE>(x, scale, shift, N, C, len, sx, alpha, out, w_curv, b_curv,
                                     (int)blockIdx.x, rowsum, prod);
}

// The backward half of the BatchNorm curvature for MANY layers in one launch: a workgroup
// takes one channel of one layer (found by binary search in the table of first items; the
// layers with the longest rows first).  Rows of up to 1024 elements run the code of
// bn_rows_kernel; longer rows are walked by one wave per sample, 8 loads in flight per lane.
struct BnJob {
  const float* g;
  const float* sx;
  float* w_curv;
  float* b_curv;
  int N, C, len, variant;       // variant: 2 * log2(chunks) + vec for short rows, 6: long rows
  float alpha;
  int pad;
};
constexpr int BN_LONG = 6;

__global__ __launch_bounds__(256) void bn_grouped_kernel(const BnJob* __restrict__ jobs,
                                                         const int* __restrict__ cum, int njobs) {
  __shared__ float rowsum[BN_MAX_ROWS];
  __shared__ float prod[BN_MAX_ROWS];
  int lo = 0, hi = njobs;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cum[mid] <= (int)blockIdx.x) lo = mid; else hi = mid;
  }
  const BnJob jb = jobs[lo];
  const int c = (int)blockIdx.x - cum[lo];
#define KFAC_BN_BODY(CH, V)                                                                   \
  bn_rows_body<CH, V, true>(jb.g, nullptr, nullptr, jb.N, jb.C, jb.len, jb.sx, jb.alpha, nullptr, \
                            jb.w_curv, jb.b_curv, c, rowsum, prod)
  switch (jb.variant) {
    case 0: KFAC_BN_BODY(1, false); return;
    case 1: KFAC_BN_BODY(1, true); return;
    case 2: KFAC_BN_BODY(2, false); return;
    case 3: KFAC_BN_BODY(2, true); return;
    case 4: KFAC_BN_BODY(4, false); return;
    case 5: KFAC_BN_BODY(4, true); return;
    default: break;
  }
#undef KFAC_BN_BODY
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int len = jb.len;
  const bool vec = (len & 3) == 0 && ((uintptr_t)jb.g & 15) == 0;
  for (int q = wave; q < jb.N; q += 4) {
    const float* p = jb.g + ((long)q * jb.C + c) * len;
    float s = 0.f;
    if (vec) {
      const float4* p4 = reinterpret_cast<const float4*>(p);
      const int len4 = len >> 2;
      for (int i = lane; i < len4; i += 64 * 8) {
        float4 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
          v[k] = i + 64 * k < len4 ? p4[i + 64 * k] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int k = 0; k < 8; ++k) s += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
      }
    } else {
      for (int i = lane; i < len; i += 64 * 8) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = i + 64 * k < len ? p[i + 64 * k] : 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) s += v[k] * v[k];
      }
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) s += __shfl_xor(s, m);
    if (lane == 0) rowsum[q] = s;
  }
  bn_finish_channel(rowsum, prod, jb.sx, jb.N, jb.C, c, jb.alpha, jb.w_curv, jb.b_curv);
}

// Launch of bn_rows_kernel when the shape suits it (false: the caller takes the
// general kernels).
template <bool COMBINE>
static bool launch_bn_rows(const float* x, const float* scale, const float* shift, int N, int C,
                           int len, const float* sx, float alpha, float* out, float* w_curv,
                           float* b_curv, hipStream_t stream) {
  const bool vec = (len & 3) == 0 && ((uintptr_t)x & 15) == 0;
  const int units = vec ? len >> 2 : len;
  if (units > 256 || N > BN_MAX_ROWS) return false;
  const int chunks = units <= 64 ? 1 : (units <= 128 ? 2 : 4);
  const dim3 grid(C), block(256);
#define KFAC_BN_ROWS(CH, V)                                                                  \
  hipLaunchKernelGGL((bn_rows_kernel<CH, V, COMBINE>), grid, block, 0, stream, x, scale, shift, \
                     N, C, len, sx, alpha, out, w_curv, b_curv)
  if (vec) {
    if (chunks == 1) KFAC_BN_ROWS(1, true);
    else if (chunks == 2) KFAC_BN_ROWS(2, true);
    else KFAC_BN_ROWS(4, true);
  } else {
    if (chunks == 1) KFAC_BN_ROWS(1, false);
    else if (chunks == 2) KFAC_BN_ROWS(2, false);
    else KFAC_BN_ROWS(4, false);
  }
#undef KFAC_BN_ROWS
  return true;
}

}  // namespace kfac

using namespace kfac;

extern "C" {

size_t kfac_vector_workspace_bytes(int count) { return count > 0 ? vec_workspace(count) : 0; }

int kfac_axpby_batched(int count, const int64_t* numel, const float* const* x, float* const* y,
                       float a, float b, void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!numel || !x || !y))) return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !x[i] || !y[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)x[i], y[i], nullptr, (long)numel[i], a, b, 0.f, 0.f};
  }
  return run_axpby(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_diag_inverse_batched(int count, const int64_t* numel, const float* const* ema,
                              float* const* inv, const float* damping, int use_sqrt,
                              void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!numel || !ema || !inv || !damping))) return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !ema[i] || !inv[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)ema[i], inv[i], nullptr, (long)numel[i], damping[i],
                   use_sqrt ? 1.f : 0.f, 0.f, 0.f};
  }
  return run_vec<OP_DIAG_INV>(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_diag_precondition_batched(int count, const int64_t* numel, const float* const* inv,
                                   float* const* grad, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  if (count < 0 || (count > 0 && (!numel || !inv || !grad))) return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !inv[i] || !grad[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)inv[i], grad[i], nullptr, (long)numel[i], 0.f, 0.f, 0.f, 0.f};
  }
  return run_vec<OP_MUL>(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_sqrt_batched(int count, const int64_t* numel, const float* const* x, float* const* y,
                       void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!numel || !x || !y))) return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !x[i] || !y[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)x[i], y[i], nullptr, (long)numel[i], 0.f, 0.f, 0.f, 0.f};
  }
  return run_vec<OP_SQRT>(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_max_batched(int count, const int64_t* numel, const float* const* x, float* const* y,
                     void* workspace, size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!numel || !x || !y))) return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !x[i] || !y[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)x[i], y[i], nullptr, (long)numel[i], 0.f, 0.f, 0.f, 0.f};
  }
  return run_vec<OP_MAX>(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_diag_sample_batched(int count, const int64_t* numel, const float* const* mean,
                             const float* const* std_dev, float* const* noise_to_param,
                             const float* std_scale, void* workspace, size_t workspace_bytes,
                             void* stream) {
  if (count < 0 || (count > 0 && (!numel || !mean || !std_dev || !noise_to_param || !std_scale)))
    return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !mean[i] || !std_dev[i] || !noise_to_param[i]) return KFAC_ERR_ARG;
    d[i] = VecDesc{(float*)mean[i], noise_to_param[i], (float*)std_dev[i], (long)numel[i],
                   std_scale[i], 0.f, 0.f, 0.f};
  }
  return run_vec<OP_ADDCMUL>(d, workspace, workspace_bytes, (hipStream_t)stream);
}

int kfac_sgd_update_batched(int count, const int64_t* numel, float* const* param,
                            float* const* grad, float* const* momentum_buf, const float* lr,
                            const float* momentum, const float* weight_decay, void* workspace,
                            size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!numel || !param || !grad || !lr || !momentum || !weight_decay)))
    return KFAC_ERR_ARG;
  std::vector<VecDesc> d(count);
  for (int i = 0; i < count; ++i) {
    if (numel[i] <= 0 || !param[i] || !grad[i]) return KFAC_ERR_ARG;
    if (momentum[i] != 0.f && (!momentum_buf || !momentum_buf[i])) return KFAC_ERR_ARG;
    d[i] = VecDesc{param[i], grad[i], momentum_buf ? momentum_buf[i] : nullptr, (long)numel[i],
                   lr[i], momentum[i], weight_decay[i], 0.f};
  }
  // float4 kernel for the tensors that allow it (the weights), scalar for the rest
  if (count == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < vec_workspace(count)) return KFAC_ERR_WORKSPACE;
  std::vector<VecDesc> v4, sc;
  for (const VecDesc& e : d) {
    const bool aligned =
        (((uintptr_t)e.a | (uintptr_t)e.b | (uintptr_t)e.c) & 15) == 0 && (e.numel & 3) == 0;
    (aligned ? v4 : sc).push_back(e);
  }
  VecDesc* table = (VecDesc*)workspace;
  if (!v4.empty()) {
    const long maxblocks = upload_table(v4, table, 4L * EW_THREADS * 2, (hipStream_t)stream);
    long gx = std::max<long>(64, 8192 / (long)v4.size());
    gx = std::min(gx, maxblocks);
    hipLaunchKernelGGL(sgd4_kernel, dim3((unsigned)gx, (unsigned)v4.size()), dim3(EW_THREADS), 0,
                       (hipStream_t)stream, table);
  }
  if (!sc.empty()) {
    VecDesc* t2 = table + v4.size();
    const long maxblocks = upload_table(sc, t2, EW_BLOCK, (hipStream_t)stream);
    long gx = std::max<long>(64, 4096 / (long)sc.size());
    gx = std::min(gx, maxblocks);
    hipLaunchKernelGGL((vec_kernel<OP_SGD>), dim3((unsigned)gx, (unsigned)sc.size()),
                       dim3(EW_THREADS), 0, (hipStream_t)stream, t2);
  }
  return launch_status();
}

static void launch_rowsq(const float* x, int64_t rows, int channels, int len, const float* scale,
                         const float* shift, float* out, hipStream_t stream) {
  if (rows % channels == 0 && rows / channels <= INT_MAX &&
      launch_bn_rows<false>(x, scale, shift, (int)(rows / channels), channels, len, nullptr, 0.f,
                            out, nullptr, nullptr, stream))
    return;
  if (len <= 256)
    hipLaunchKernelGGL(rowsq_kernel<4>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, x,
                       scale, shift, (long)rows, channels, len, out);
  else
    hipLaunchKernelGGL(rowsq_kernel<1>, dim3((unsigned)rows), dim3(256), 0, stream, x, scale,
                       shift, (long)rows, channels, len, out);
}

int kfac_rowsq_sum(const float* x, int64_t rows, int channels, int len, const float* scale,
                   const float* shift, float* out, void* stream) {
  if (!x || !out || rows <= 0 || channels <= 0 || len <= 0 || rows >= (int64_t)1 << 31)
    return KFAC_ERR_ARG;
  launch_rowsq(x, rows, channels, len, scale, shift, out, (hipStream_t)stream);
  return launch_status();
}

size_t kfac_bn_diag_cov_workspace_bytes(int n, int channels) {
  return n > 0 && channels > 0 ? (size_t)n * channels * sizeof(float) : 0;
}

int kfac_bn_diag_cov(const float* g, int n, int channels, int len, const float* sx, float alpha,
                     float* w_curv, float* b_curv, void* workspace, size_t workspace_bytes,
                     void* stream) {
  if (!g || !sx || !w_curv || n <= 0 || channels <= 0 || len <= 0 ||
      (int64_t)n * channels >= (int64_t)1 << 31)
    return KFAC_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (launch_bn_rows<true>(g, nullptr, nullptr, n, channels, len, sx, alpha, nullptr, w_curv,
                           b_curv, st))
    return launch_status();
  if (!workspace || workspace_bytes < kfac_bn_diag_cov_workspace_bytes(n, channels))
    return KFAC_ERR_WORKSPACE;
  float* sg = (float*)workspace;
  launch_rowsq(g, (int64_t)n * channels, channels, len, nullptr, nullptr, sg, st);
  hipLaunchKernelGGL(bn_combine_kernel, dim3(cdiv(channels, 64)), dim3(256), 0, st, sx, sg, n,
                     channels, alpha, w_curv, b_curv);
  return launch_status();
}

size_t kfac_bn_diag_cov_batched_workspace_bytes(int count) {
  if (count <= 0) return 0;
  return (((size_t)count * sizeof(BnJob) + 255) & ~(size_t)255) + ((size_t)count + 1) * sizeof(int);
}

int kfac_bn_diag_cov_batched(int count, const float* const* g, const int* n, const int* channels,
                             const int* len, const float* const* sx, const float* alpha,
                             float* const* w_curv, float* const* b_curv, void* workspace,
                             size_t workspace_bytes, void* stream) {
  if (count < 0 || (count > 0 && (!g || !n || !channels || !len || !sx || !alpha || !w_curv)))
    return KFAC_ERR_ARG;
  if (count == 0) return KFAC_OK;
  if (!workspace || workspace_bytes < kfac_bn_diag_cov_batched_workspace_bytes(count))
    return KFAC_ERR_WORKSPACE;
  long items = 0;
  for (int i = 0; i < count; ++i) {
    if (!g[i] || !sx[i] || !w_curv[i] || n[i] <= 0 || n[i] > BN_MAX_ROWS || channels[i] <= 0 ||
        len[i] <= 0 || (int64_t)n[i] * channels[i] >= (int64_t)1 << 31)
      return KFAC_ERR_ARG;
    items += channels[i];
  }
  if (items >= (long)1 << 31) return KFAC_ERR_ARG;
  // the layers with the longest rows first: their workgroups last longest
  std::vector<int> order(count);
  for (int i = 0; i < count; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
    return (long)len[a] * n[a] > (long)len[b] * n[b];
  });
  const size_t jobs_bytes = ((size_t)count * sizeof(BnJob) + 255) & ~(size_t)255;
  std::vector<unsigned> words((jobs_bytes + ((size_t)count + 1) * sizeof(int)) / 4, 0u);
  BnJob* jobs = (BnJob*)words.data();
  int* cum = (int*)((char*)words.data() + jobs_bytes);
  int at = 0;
  for (int k = 0; k < count; ++k) {
    const int i = order[k];
    const bool vec = (len[i] & 3) == 0 && ((uintptr_t)g[i] & 15) == 0;
    const int units = vec ? len[i] >> 2 : len[i];
    const int variant = units > 256 ? BN_LONG
                                    : 2 * (units <= 64 ? 0 : (units <= 128 ? 1 : 2)) + (vec ? 1 : 0);
    jobs[k] = BnJob{g[i], sx[i], w_curv[i], b_curv ? b_curv[i] : nullptr, n[i], channels[i],
                    len[i], variant, alpha[i], 0};
    cum[k] = at;
    at += channels[i];
  }
  cum[count] = at;
  hipStream_t st = (hipStream_t)stream;
  upload_table(words.data(), words.size() * 4, workspace, st);
  hipLaunchKernelGGL(bn_grouped_kernel, dim3(at), dim3(256), 0, st, (const BnJob*)workspace,
                     (const int*)((char*)workspace + jobs_bytes), count);
  return launch_status();
}

int kfac_scale_rows(const float* x, const float* w, int64_t rows, int64_t len, int use_sqrt,
                    float* out, void* stream) {
  if (!x || !w || !out || rows <= 0 || len <= 0) return KFAC_ERR_ARG;
  const long total = (long)rows * len;
  long blocks = (total + 1023) / 1024;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(scale_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     x, w, (long)rows, (long)len, use_sqrt, out);
  return launch_status();
}

int kfac_bn_diag_combine(const float* sx, const float* sg, int n, int channels, float alpha,
                         float* w_curv, float* b_curv, void* stream) {
  if (!sx || !sg || !w_curv || n <= 0 || channels <= 0) return KFAC_ERR_ARG;
  hipLaunchKernelGGL(bn_combine_kernel, dim3(cdiv(channels, 64)), dim3(256), 0,
                     (hipStream_t)stream, sx, sg, n, channels, alpha, w_curv, b_curv);
  return launch_status();
}

}  // extern "C"
