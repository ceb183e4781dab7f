// Grouped Kronecker factor build: the symmetric products of MANY layers in a handful of
// launches.
//
// A factor product depends only on the tensor its hook was handed and nothing reads it
// before the optimizer step, so the host may collect the products of a whole
// forward / backward pass and hand them over together.  One launch per operand kind
// and tile configuration then holds the (tile, k-split) work items of all its products,
// longest first: a launch of thousands of items keeps every CU busy until its end,
// where a launch per product (a few hundred items, often fewer) drains and refills the
// chip a hundred times per step; the k-split partials of all products are reduced by
// two more launches at the end instead of one or two per product.
//
//   work item -> product: binary search in the table of first items (uniform per
//   workgroup, scalar loads); inside a product the items are renumbered so that each
//   XCD (own L2) walks a contiguous run of (split, tile) pairs, tile fastest, as in
//   the single-product kernel.
//
// The input factor of a convolution that is not pointwise reads a copy of its input:
// zero-padded, one plane per row phase of the stride and per kernel column
// (conv_planes_kernel, one launch for all such products of the call).  The operand then
// needs no bounds test and reads consecutive addresses along the reduction.
//
// Products whose input exceeds the 1 GiB addressing window of an operand, and the
// stride-1 k x k layers served by the correlation kernels, are handed to their
// single-product routines on the same stream.
#include <string.h>

#include <algorithm>
#include <type_traits>
#include <vector>

#include "common.h"
#include "operands.h"
#include "syrk_reduce.h"

namespace kfac {

// ---- device tables -----------------------------------------------------------

template <class OP>
struct SyJob {
  OP op;
  float* C;
  const float* Cin;
  float* ws;            // partials of this product (splits > 1)
  int d, K, T, ntiles, splits, cps;
  float alpha, beta;
};

struct RdJob {
  const float* ws;
  float* C;
  const float* Cin;
  int d, T, ntiles, splits;
  float alpha, beta;
};

// first table entry whose range holds `item` (cum[j] <= item < cum[j + 1])
__device__ __forceinline__ int find_job(const int* __restrict__ cum, int njobs, int item) {
  int lo = 0, hi = njobs;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cum[mid] <= item) lo = mid; else hi = mid;
  }
  return lo;
}

template <class OP, int W>
__global__ __launch_bounds__(64 * W * W, W == 2 ? 3 : 1) void syrk_grouped_kernel(
    const SyJob<OP>* __restrict__ jobs, const int* __restrict__ cum, int njobs) {
  constexpr int TS = 64 * W;
  constexpr int KC = Cfg<W, W>::KC;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int g = blockIdx.x;
  const int j = find_job(cum, njobs, g);
  const SyJob<OP>& jb = jobs[j];
  const int c0 = cum[j];
  const int ntiles = jb.ntiles, splits = jb.splits;
  const int item = xcd_remap_range(g, c0, ntiles * splits);
  const int tile = item % ntiles;
  const int split = item / ntiles;
  int bi, bj;
  upper_tile(tile, jb.T, bi, bj);
  const int K = jb.K, d = jb.d;
  const int kbeg = split * jb.cps * KC;
  int kend = kbeg + jb.cps * KC;
  if (kend > K) kend = K;
  const OP op = jb.op;
  if (splits == 1) {
    EpiStore epi{jb.C, d, d, d, jb.alpha, jb.beta, bi != bj, jb.Cin};
    gemm_tile_cfg<W, W, true>(op, op, bi * TS, bj * TS, kbeg, kend, bi == bj, epi, smem);
  } else {
    EpiPartial epi{jb.ws + ((size_t)split * ntiles + tile) * (TS * TS), bi * TS, bj * TS, d, d, TS};
    gemm_tile_cfg<W, W, true>(op, op, bi * TS, bj * TS, kbeg, kend, bi == bj, epi, smem);
  }
}

// many splits: item = (tile, row of the tile, 64-wide segment)
template <int TS>
__global__ __launch_bounds__(256) void reduce_many_grouped_kernel(const RdJob* __restrict__ jobs,
                                                                  const int* __restrict__ cum,
                                                                  int njobs) {
  const int j = find_job(cum, njobs, blockIdx.x);
  const RdJob jb = jobs[j];
  const int local = blockIdx.x - cum[j];
  constexpr int PER_TILE = TS * (TS / 64);
  const int tile = local / PER_TILE;
  syrk_reduce_many<TS>(jb.ws, jb.d, jb.T, jb.ntiles, jb.splits, jb.C, jb.Cin, jb.alpha, jb.beta,
                       tile, local - tile * PER_TILE);
}

// few splits: item = (tile, 32-row block, 64-column block)
template <int TS>
__global__ __launch_bounds__(256) void reduce_tile_grouped_kernel(const RdJob* __restrict__ jobs,
                                                                  const int* __restrict__ cum,
                                                                  int njobs) {
  const int j = find_job(cum, njobs, blockIdx.x);
  const RdJob jb = jobs[j];
  const int local = blockIdx.x - cum[j];
  constexpr int CB = TS / 64, PER_TILE = (TS / 32) * CB;
  const int tile = local / PER_TILE;
  const int rem = local - tile * PER_TILE;
  syrk_reduce_tile<TS>(jb.ws, jb.d, jb.T, jb.ntiles, jb.splits, jb.C, jb.Cin, jb.alpha, jb.beta,
                       tile, rem / CB, rem % CB);
}

// One convolution input and its copy in planes (see ConvP).  Only the row phases that
// some kernel tap reads are written (a 1x1 convolution of stride 2 reads one of two).
constexpr int MAX_PLANES = 32;
constexpr int PLANE_ITEM = 8192;      // elements of the copy per workgroup
struct PlaneJob {
  const float* x;
  float* out;
  int C, H, W, sh, sw, ph, pw, dw, KW, Hs, OW, nused, chunks, ones, image;
  FastDiv by_ow, by_area, by_chunks, by_c;
  unsigned char used[MAX_PLANES];     // ry * KW + kw of the planes to write
};

// item = (channel image (n, c), chunk of its used planes): PLANE_ITEM elements, in order
__global__ __launch_bounds__(256) void conv_planes_kernel(const PlaneJob* __restrict__ jobs,
                                                          const int* __restrict__ cum, int njobs) {
  const int j = find_job(cum, njobs, blockIdx.x);
  const PlaneJob& jb = jobs[j];
  const int local = blockIdx.x - cum[j];
  const int img = jb.by_chunks.div(local);
  const int chunk = local - img * jb.chunks;
  const int n = jb.by_c.div(img), c = img - n * jb.C;
  const int H = jb.H, W = jb.W, OW = jb.OW, area = jb.Hs * OW, planes = jb.sh * jb.KW;
  const float* __restrict__ src = jb.x + (size_t)img * H * W;
  float* __restrict__ dst = jb.out + (size_t)n * jb.image + (size_t)c * planes * area;
  const int total = jb.nused * area;
  const int e1 = min(total, (chunk + 1) * PLANE_ITEM);
  // four elements per thread and trip, so that four loads are in flight
  for (int e0 = chunk * PLANE_ITEM + threadIdx.x; e0 < e1; e0 += 4 * 256) {
    float v[4];
    int at[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = e0 + 256 * q;
      const int u = jb.by_area.div(e);
      const int idx = e - u * area;
      const int plane = jb.used[u & (MAX_PLANES - 1)];
      const int ry = plane / jb.KW, kw = plane - ry * jb.KW;
      const int ys = jb.by_ow.div(idx);
      const int ow = idx - ys * OW;
      const int y = ys * jb.sh + ry - jb.ph, x = ow * jb.sw + kw * jb.dw - jb.pw;
      const bool in = e < e1 && (unsigned)y < (unsigned)H && (unsigned)x < (unsigned)W;
      at[q] = e < e1 ? plane * area + idx : -1;
      v[q] = in ? src[y * W + x] : 0.f;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (at[q] >= 0) dst[at[q]] = v[q];
  }
  if (jb.ones && c == 0 && chunk == 0) {
    float* __restrict__ one = jb.out + (size_t)n * jb.image + (size_t)jb.C * planes * area;
    for (int idx = threadIdx.x; idx < jb.ones; idx += 256) one[idx] = 1.f;
  }
}

// ---- host side -----------------------------------------------------------------

// Items of a grouped launch are dispatched longest first and the launch holds many of
// them, so an item may be long: about this many 16-deep chunks, which keeps the
// partial tiles that a split writes and the reduction reads small beside the input.
constexpr int GROUP_TARGET_CPS_W2 = 96;
constexpr int GROUP_TARGET_CPS_W1 = 192;
constexpr int MANY_SPLITS = 16;          // above: the reduction with 16 split lanes

struct GroupPlan {
  int w, ts, T, ntiles, splits, cps;
  size_t partial_floats() const {
    return splits > 1 ? (size_t)splits * ntiles * ts * ts : 0;
  }
};

// 64-wide tiles (one wave each) up to 192 rows; from there a 128-wide tile has at most a
// quarter of padding and loads half as many operand elements per matrix instruction
// (factors of 256 rows: 7 % faster on 128-wide tiles).
constexpr int GROUP_W1_MAX_DIM = 192;

static GroupPlan plan_group(int d, long K, long target) {
  GroupPlan p;
  p.w = d <= GROUP_W1_MAX_DIM ? 1 : 2;
  p.ts = 64 * p.w;
  p.T = cdiv(d, p.ts);
  p.ntiles = p.T * (p.T + 1) / 2;
  const long nchunks = (K + 15) / 16;
  long splits = (nchunks + target / 2) / target;
  if (splits < 1) splits = 1;
  long cps = (nchunks + splits - 1) / splits;
  splits = (nchunks + cps - 1) / cps;
  p.splits = (int)splits;
  p.cps = (int)cps;
  return p;
}

// Chunks per item for one launch: the default when the launch holds plenty of items at that
// length, shorter items when it would not fill the chip twice (resident workgroups: 3 per CU
// of four waves, 8 per CU of one wave).
static long launch_target(int w, double total_units) {
  const long dflt = w == 1 ? GROUP_TARGET_CPS_W1 : GROUP_TARGET_CPS_W2;
  const double slots = w == 1 ? 2048. : 768.;
  long t = (long)(total_units / (2. * slots));
  if (t > dflt) t = dflt;
  if (t < 8) t = 8;
  return t;
}

enum Path { P_DENSE, P_CONVG, P_CONVA, P_CONVP, P_TAPS, P_SINGLE, P_BAD };
constexpr int SYRK_PATHS = 4;     // the first four: one launch each per tile size

struct Classified {
  Path path;
  int d;
  long K;
  int OH, OW;
  int Hs;                // P_CONVP: rows of a plane of the copy
  size_t copy_bytes;     // P_CONVP: 0 when the input itself serves
};

static Classified classify(const kfac_factor_job& j) {
  Classified c{P_BAD, 0, 0, 0, 0, 0, 0};
  if (j.rows <= 0 || j.c <= 0) return c;
  const int bias = j.add_bias ? 1 : 0;
  if (j.kind == KFAC_FACTOR_LINEAR) {
    c.d = j.c + bias;
    c.K = j.rows;
    if ((int64_t)c.d * c.d * 4 > MAX_OPERAND_BYTES) return c;
    c.path = (int64_t)j.rows * j.c * 4 <= MAX_OPERAND_BYTES ? P_DENSE : P_SINGLE;
    return c;
  }
  if (j.rows > INT32_MAX || j.H <= 0 || j.W <= 0) return c;
  const int64_t tensor_bytes = (int64_t)j.rows * j.c * j.H * j.W * 4;
  if (j.kind == KFAC_FACTOR_CONV_G) {
    c.d = j.c;
    c.K = (long)j.rows * j.H * j.W;
    if ((int64_t)c.d * c.d * 4 > MAX_OPERAND_BYTES) return c;
    c.path = tensor_bytes <= MAX_OPERAND_BYTES && c.K <= INT32_MAX ? P_CONVG : P_SINGLE;
    return c;
  }
  if (j.kind != KFAC_FACTOR_CONV_A) return c;
  if (j.kh <= 0 || j.kw <= 0 || j.sh <= 0 || j.sw <= 0 || j.ph < 0 || j.pw < 0 || j.dh <= 0 ||
      j.dw <= 0)
    return c;
  if (j.H >= 16384 || j.W >= 16384 || j.kh * j.dh >= 16384 || j.kw * j.dw >= 16384) return c;
  c.OH = (j.H + 2 * j.ph - j.dh * (j.kh - 1) - 1) / j.sh + 1;
  c.OW = (j.W + 2 * j.pw - j.dw * (j.kw - 1) - 1) / j.sw + 1;
  if (c.OH <= 0 || c.OW <= 0) return c;
  const int64_t dd = (int64_t)j.c * j.kh * j.kw + bias;
  if (dd * dd * 4 > MAX_OPERAND_BYTES) return c;
  c.d = (int)dd;
  c.K = (long)j.rows * c.OH * c.OW;
  if (tensor_bytes > MAX_OPERAND_BYTES || c.K > INT32_MAX) {
    c.path = P_SINGLE;
  } else if (j.kh == 1 && j.kw == 1 && j.sh == 1 && j.sw == 1 && j.ph == 0 && j.pw == 0 && !bias) {
    c.path = P_CONVG;          // a pointwise convolution: M is the input viewed as [c, n*H*W]
  } else if (conv_a_taps_applicable(j.c, j.kh, j.kw, j.sh, j.sw, bias) &&
             conv_a_taps_workspace((int)j.rows, j.c, j.H, j.W, j.kh, j.kw, j.ph, j.pw, j.dh,
                                   j.dw) > 0) {
    c.path = P_TAPS;
  } else {
    c.path = P_CONVA;
    // the copy in planes, where it fits the addressing window of an operand
    c.Hs = c.OH + (j.kh - 1) * j.dh / j.sh;
    const int64_t copy =
        j.rows * ((int64_t)j.c * j.sh * j.kw * c.Hs * c.OW + (bias ? c.OH * c.OW : 0)) * 4;
    // (a pointwise convolution with a stride reads so little per product that the copy
    // costs more than the bounds tests)
    if (j.kh * j.kw > 1 && j.sh * j.kw <= MAX_PLANES && copy <= MAX_OPERAND_BYTES) {
      c.path = P_CONVP;
      // (a k x 1 kernel, stride 1, no padding, no bias: one plane, Hs = H, OW = W)
      const bool as_is =
          j.sh == 1 && j.sw == 1 && j.ph == 0 && j.pw == 0 && j.kw == 1 && !bias;
      c.copy_bytes = as_is ? 0 : (size_t)copy;
    }
  }
  return c;
}

static size_t single_workspace(const kfac_factor_job& j, const Classified& c) {
  if (j.kind == KFAC_FACTOR_CONV_A)
    return kfac_factor_conv_a_workspace_bytes((int)j.rows, j.c, j.H, j.W, j.kh, j.kw, j.sh, j.sw,
                                              j.ph, j.pw, j.dh, j.dw, j.add_bias ? 1 : 0);
  // (linear / conv G in slices: the largest slice is the whole reduction at most)
  return kfac_factor_workspace_bytes(c.d, c.K);
}

static int run_single(const kfac_factor_job& j, void* ws, size_t ws_bytes, void* stream) {
  switch (j.kind) {
    case KFAC_FACTOR_LINEAR:
      return kfac_factor_linear(j.x, j.rows, j.c, j.c, j.add_bias, j.alpha, j.beta, j.C_prev, j.C,
                                ws, ws_bytes, stream);
    case KFAC_FACTOR_CONV_G:
      return kfac_factor_conv_g(j.x, (int)j.rows, j.c, j.H, j.W, j.alpha, j.beta, j.C_prev, j.C, ws,
                                ws_bytes, stream);
    default:
      return kfac_factor_conv_a(j.x, (int)j.rows, j.c, j.H, j.W, j.kh, j.kw, j.sh, j.sw, j.ph,
                                j.pw, j.dh, j.dw, j.add_bias, j.alpha, j.beta, j.C_prev, j.C, ws,
                                ws_bytes, stream);
  }
}

static size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// The whole plan of a grouped call: which path every product takes, where its partials
// live, and the device tables of the launches.
struct GroupedPlan {
  bool ok = true;
  std::vector<Classified> cls;
  std::vector<GroupPlan> plans;         // syrk paths only
  std::vector<size_t> partial_off;      // floats, from the partial area
  size_t table_bytes = 0, partial_floats = 0, single_bytes = 0;
  double executed_flops = 0.;
  // members of each launch, longest items first
  std::vector<int> members[SYRK_PATHS][2];   // [P_DENSE | P_CONVG | P_CONVA | P_CONVP][w - 1]
  std::vector<size_t> copy_off;         // P_CONVP with a copy: bytes, from the copy area
  std::vector<int> copies;              // the products that read a copy
  size_t copy_bytes = 0;
  std::vector<int> reduce_many[2], reduce_tile[2];   // [w - 1]
  std::vector<int> singles;             // P_SINGLE, in call order
  std::vector<int> taps;                // P_TAPS, in call order
  size_t taps_bytes = 0;
};

template <class T>
static size_t table_size(size_t n) {
  return n ? align_up(n * sizeof(T), 16) + align_up((n + 1) * sizeof(int), 16) : 0;
}

static std::vector<TapsJob> taps_jobs(const GroupedPlan& gp, const kfac_factor_job* jobs) {
  std::vector<TapsJob> tj;
  for (int i : gp.taps) {
    const kfac_factor_job& j = jobs[i];
    tj.push_back(TapsJob{j.x, (int)j.rows, j.c, j.H, j.W, j.kh, j.kw, j.ph, j.pw, j.dh, j.dw,
                         j.alpha, j.beta, j.C_prev, j.C});
  }
  return tj;
}

static GroupedPlan make_plan(int count, const kfac_factor_job* jobs) {
  GroupedPlan gp;
  gp.cls.resize(count);
  gp.plans.resize(count);
  gp.partial_off.assign(count, 0);
  gp.copy_off.assign(count, 0);
  for (int i = 0; i < count; ++i) {
    const Classified c = classify(jobs[i]);
    gp.cls[i] = c;
    if (c.path == P_BAD) {
      gp.ok = false;
      return gp;
    }
    if (c.path == P_TAPS) {
      gp.taps.push_back(i);
      continue;
    }
    if (c.path == P_SINGLE) {
      gp.singles.push_back(i);
      gp.single_bytes = std::max(gp.single_bytes, single_workspace(jobs[i], c));
      const kfac_factor_job& j = jobs[i];
      gp.executed_flops +=
          j.kind == KFAC_FACTOR_CONV_A
              ? kfac_factor_conv_a_executed_flops((int)j.rows, j.c, j.H, j.W, j.kh, j.kw, j.sh,
                                                  j.sw, j.ph, j.pw, j.dh, j.dw, j.add_bias ? 1 : 0)
              : kfac_factor_executed_flops(c.d, c.K);
      continue;
    }
    const int w = c.d <= GROUP_W1_MAX_DIM ? 1 : 2;
    gp.members[c.path][w - 1].push_back(i);
    if (c.path == P_CONVP && c.copy_bytes) {
      gp.copies.push_back(i);
      gp.copy_off[i] = gp.copy_bytes;
      gp.copy_bytes += align_up(c.copy_bytes, 256);
    }
  }
  for (int path = 0; path < SYRK_PATHS; ++path)
    for (int w = 0; w < 2; ++w) {
      double units = 0.;
      for (int i : gp.members[path][w]) {
        const int T = cdiv(gp.cls[i].d, 64 * (w + 1));
        units += (double)(T * (T + 1) / 2) * (double)((gp.cls[i].K + 15) / 16);
      }
      const long target = launch_target(w + 1, units);
      for (int i : gp.members[path][w]) {
        const Classified& c = gp.cls[i];
        const GroupPlan p = plan_group(c.d, c.K, target);
        gp.plans[i] = p;
        gp.partial_off[i] = gp.partial_floats;
        gp.partial_floats += p.partial_floats();
        if (p.splits > MANY_SPLITS)
          gp.reduce_many[w].push_back(i);
        else if (p.splits > 1)
          gp.reduce_tile[w].push_back(i);
        gp.executed_flops +=
            syrk_tile_units(p.T, p.w) * (double)((c.K + 15) / 16) * 16 * 2.0 * p.ts * p.ts;
      }
    }
  for (int path = 0; path < SYRK_PATHS; ++path)
    for (int w = 0; w < 2; ++w) {
      auto& m = gp.members[path][w];
      std::stable_sort(m.begin(), m.end(),
                       [&](int a, int b) { return gp.plans[a].cps > gp.plans[b].cps; });
    }
  for (int w = 0; w < 2; ++w) {
    gp.table_bytes += table_size<SyJob<DenseKM>>(gp.members[P_DENSE][w].size());
    gp.table_bytes += table_size<SyJob<ConvG>>(gp.members[P_CONVG][w].size());
    gp.table_bytes += table_size<SyJob<ConvA>>(gp.members[P_CONVA][w].size());
    gp.table_bytes += table_size<SyJob<ConvP>>(gp.members[P_CONVP][w].size());
    gp.table_bytes += table_size<RdJob>(gp.reduce_many[w].size());
    gp.table_bytes += table_size<RdJob>(gp.reduce_tile[w].size());
  }
  gp.table_bytes += table_size<PlaneJob>(gp.copies.size());
  gp.table_bytes = align_up(gp.table_bytes, 256);
  if (!gp.taps.empty()) {
    const std::vector<TapsJob> tj = taps_jobs(gp, jobs);
    gp.taps_bytes = align_up(conv_a_taps_grouped_workspace((int)tj.size(), tj.data()), 256);
    gp.executed_flops += conv_a_taps_grouped_executed_flops((int)tj.size(), tj.data());
  }
  return gp;
}

// The plan depends on the shapes only, and a training loop hands over the same few lists
// step after step: the last plans of every host thread are kept (never freed: objects of
// this library have no destructors that could run at process exit).
struct JobShape {
  int64_t rows;
  int kind, add_bias, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, unused;
  bool operator==(const JobShape& o) const { return memcmp(this, &o, sizeof(JobShape)) == 0; }
};
static_assert(sizeof(JobShape) == sizeof(int64_t) + 14 * sizeof(int),
              "no padding: the shapes are compared as bytes");

static JobShape shape_of(const kfac_factor_job& j) {
  JobShape s;
  memset(&s, 0, sizeof(s));
  s.kind = j.kind;
  s.add_bias = j.add_bias ? 1 : 0;
  s.c = j.c;
  s.H = j.kind == KFAC_FACTOR_LINEAR ? 0 : j.H;
  s.W = j.kind == KFAC_FACTOR_LINEAR ? 0 : j.W;
  if (j.kind == KFAC_FACTOR_CONV_A) {
    s.kh = j.kh; s.kw = j.kw; s.sh = j.sh; s.sw = j.sw;
    s.ph = j.ph; s.pw = j.pw; s.dh = j.dh; s.dw = j.dw;
  }
  s.rows = j.rows;
  return s;
}

struct CachedPlan {
  std::vector<JobShape> shapes;
  GroupedPlan plan;
};

static const GroupedPlan& cached_plan(int count, const kfac_factor_job* jobs) {
  constexpr int SLOTS = 16;
  static thread_local CachedPlan** slots = nullptr;
  static thread_local int next_slot = 0;
  if (!slots) slots = new CachedPlan*[SLOTS]();
  std::vector<JobShape> shapes((size_t)count);
  for (int i = 0; i < count; ++i) shapes[i] = shape_of(jobs[i]);
  for (int k = 0; k < SLOTS; ++k)
    if (slots[k] && slots[k]->shapes == shapes) return slots[k]->plan;
  CachedPlan* fresh = new CachedPlan{std::move(shapes), make_plan(count, jobs)};
  CachedPlan*& slot = slots[next_slot];
  next_slot = (next_slot + 1) % SLOTS;
  delete slot;
  slot = fresh;
  return slot->plan;
}

static size_t plan_workspace(const GroupedPlan& gp) {
  return gp.table_bytes + align_up(gp.partial_floats * sizeof(float), 256) + gp.taps_bytes +
         gp.single_bytes + gp.copy_bytes;
}

// host image of the device tables, filled section by section
struct TableWriter {
  std::vector<unsigned> words;
  template <class T>
  size_t put(const std::vector<T>& v, size_t align = 16) {       // returns the byte offset
    const size_t off = words.size() * 4;
    const size_t bytes = align_up(v.size() * sizeof(T), align);
    words.resize(words.size() + bytes / 4, 0u);
    memcpy((char*)words.data() + off, v.data(), v.size() * sizeof(T));
    return off;
  }
};

template <class OP>
static OP make_op(const kfac_factor_job& j, const Classified& c);

template <>
DenseKM make_op<DenseKM>(const kfac_factor_job& j, const Classified& c) {
  return DenseKM{j.x, nullptr, j.c, c.d, j.add_bias ? 1 : 0};
}
template <>
ConvG make_op<ConvG>(const kfac_factor_job& j, const Classified&) {
  return ConvG(j.x, j.c, j.H * j.W);
}
template <>
ConvA make_op<ConvA>(const kfac_factor_job& j, const Classified& c) {
  return ConvA(j.x, j.c, j.H, j.W, j.kh, j.kw, j.sh, j.sw, j.ph, j.pw, j.dh, j.dw, c.OH, c.OW, c.d,
               j.add_bias ? 1 : 0);
}

template <>
ConvP make_op<ConvP>(const kfac_factor_job& j, const Classified& c) {
  return ConvP(j.x, j.c, j.kh, j.kw, j.sh, j.dh, c.Hs, c.OH, c.OW, c.d, j.add_bias ? 1 : 0);
}

struct Launch {
  size_t jobs_off, cum_off;
  int njobs, items;
};

template <class OP>
static Launch fill_syrk(TableWriter& tw, const GroupedPlan& gp, const std::vector<int>& members,
                        const kfac_factor_job* jobs, float* partials, const char* copies) {
  if (members.empty()) return Launch{0, 0, 0, 0};
  std::vector<SyJob<OP>> tab;
  std::vector<int> cum;
  int items = 0;
  for (int i : members) {
    const GroupPlan& p = gp.plans[i];
    const kfac_factor_job& j = jobs[i];
    SyJob<OP> s;
    s.op = make_op<OP>(j, gp.cls[i]);
    if constexpr (std::is_same<OP, ConvP>::value) {
      if (gp.cls[i].copy_bytes) s.op.p = (const float*)(copies + gp.copy_off[i]);
    }
    s.C = j.C;
    s.Cin = j.C_prev;
    s.ws = partials + gp.partial_off[i];
    s.d = gp.cls[i].d;
    s.K = (int)gp.cls[i].K;
    s.T = p.T;
    s.ntiles = p.ntiles;
    s.splits = p.splits;
    s.cps = p.cps;
    s.alpha = j.alpha;
    s.beta = j.beta;
    tab.push_back(s);
    cum.push_back(items);
    items += p.ntiles * p.splits;
  }
  cum.push_back(items);
  Launch l;
  l.jobs_off = tw.put(tab);
  l.cum_off = tw.put(cum);
  l.njobs = (int)members.size();
  l.items = items;
  return l;
}

static Launch fill_reduce(TableWriter& tw, const GroupedPlan& gp, const std::vector<int>& members,
                          const kfac_factor_job* jobs, float* partials, bool many) {
  if (members.empty()) return Launch{0, 0, 0, 0};
  std::vector<RdJob> tab;
  std::vector<int> cum;
  int items = 0;
  for (int i : members) {
    const GroupPlan& p = gp.plans[i];
    const kfac_factor_job& j = jobs[i];
    tab.push_back(RdJob{partials + gp.partial_off[i], j.C, j.C_prev, gp.cls[i].d, p.T, p.ntiles,
                        p.splits, j.alpha, j.beta});
    cum.push_back(items);
    items += p.ntiles * (many ? p.ts * (p.ts / 64) : (p.ts / 32) * (p.ts / 64));
  }
  cum.push_back(items);
  Launch l;
  l.jobs_off = tw.put(tab);
  l.cum_off = tw.put(cum);
  l.njobs = (int)members.size();
  l.items = items;
  return l;
}

// the copies in planes of all products that read one
static Launch fill_planes(TableWriter& tw, const GroupedPlan& gp, const kfac_factor_job* jobs,
                          char* copies) {
  if (gp.copies.empty()) return Launch{0, 0, 0, 0};
  std::vector<PlaneJob> tab;
  std::vector<int> cum;
  int items = 0;
  for (int i : gp.copies) {
    const kfac_factor_job& j = jobs[i];
    const Classified& c = gp.cls[i];
    PlaneJob pj;
    memset(&pj, 0, sizeof(pj));
    pj.x = j.x;
    pj.out = (float*)(copies + gp.copy_off[i]);
    pj.C = j.c;
    pj.H = j.H; pj.W = j.W;
    pj.sh = j.sh; pj.sw = j.sw;
    pj.ph = j.ph; pj.pw = j.pw;
    pj.dw = j.dw; pj.KW = j.kw;
    pj.Hs = c.Hs; pj.OW = c.OW;
    bool seen[MAX_PLANES] = {};
    for (int kh = 0; kh < j.kh; ++kh) seen[kh * j.dh % j.sh] = true;
    for (int ry = 0; ry < j.sh; ++ry)
      for (int kw = 0; kw < j.kw && seen[ry]; ++kw)
        pj.used[pj.nused++] = (unsigned char)(ry * j.kw + kw);
    const int area = c.Hs * c.OW;
    pj.chunks = cdiv(pj.nused * area, PLANE_ITEM);
    pj.ones = j.add_bias ? c.OH * c.OW : 0;
    pj.image = j.c * j.sh * j.kw * area + pj.ones;
    pj.by_ow = FastDiv((unsigned)c.OW);
    pj.by_area = FastDiv((unsigned)area);
    pj.by_chunks = FastDiv((unsigned)pj.chunks);
    pj.by_c = FastDiv((unsigned)j.c);
    tab.push_back(pj);
    cum.push_back(items);
    items += (int)j.rows * j.c * pj.chunks;
  }
  cum.push_back(items);
  Launch l;
  l.jobs_off = tw.put(tab);
  l.cum_off = tw.put(cum);
  l.njobs = (int)gp.copies.size();
  l.items = items;
  return l;
}

template <class OP, int W>
static bool launch_syrk_group(const Launch& l, char* table, hipStream_t stream) {
  if (l.njobs == 0) return true;
  constexpr int lds_bytes = Cfg<W, W>::SMEM_FLOATS * (int)sizeof(float);
  if (!enable_large_lds((const void*)syrk_grouped_kernel<OP, W>, lds_bytes)) return false;
  hipLaunchKernelGGL((syrk_grouped_kernel<OP, W>), dim3(l.items), dim3(64 * W * W), lds_bytes,
                     stream, (const SyJob<OP>*)(table + l.jobs_off),
                     (const int*)(table + l.cum_off), l.njobs);
  return true;
}

}  // namespace kfac

using namespace kfac;

extern "C" {

size_t kfac_factor_grouped_workspace_bytes(int count, const kfac_factor_job* jobs) {
  if (count <= 0 || !jobs) return 0;
  const GroupedPlan& gp = cached_plan(count, jobs);
  return gp.ok ? plan_workspace(gp) : 0;
}

double kfac_factor_grouped_executed_flops(int count, const kfac_factor_job* jobs) {
  if (count <= 0 || !jobs) return 0.;
  const GroupedPlan& gp = cached_plan(count, jobs);
  return gp.ok ? gp.executed_flops : 0.;
}

int kfac_factor_grouped(int count, const kfac_factor_job* jobs, void* workspace,
                        size_t workspace_bytes, void* stream_) {
  if (count < 0 || (count > 0 && !jobs)) return KFAC_ERR_ARG;
  if (count == 0) return KFAC_OK;
  const GroupedPlan& gp = cached_plan(count, jobs);
  if (!gp.ok) return KFAC_ERR_ARG;
  for (int i = 0; i < count; ++i)
    if (!jobs[i].x || !jobs[i].C) return KFAC_ERR_ARG;
  // two products of one call must not write the same factor
  {
    std::vector<const float*> outs;
    for (int i = 0; i < count; ++i) outs.push_back(jobs[i].C);
    std::sort(outs.begin(), outs.end());
    if (std::adjacent_find(outs.begin(), outs.end()) != outs.end()) return KFAC_ERR_ARG;
  }
  const size_t need = plan_workspace(gp);
  if (need > 0 && (!workspace || workspace_bytes < need)) return KFAC_ERR_WORKSPACE;
  hipStream_t stream = (hipStream_t)stream_;
  char* table = (char*)workspace;
  float* partials = (float*)(table + gp.table_bytes);
  char* taps_ws = (char*)partials + align_up(gp.partial_floats * sizeof(float), 256);
  char* single_ws = taps_ws + gp.taps_bytes;
  char* copies = single_ws + gp.single_bytes;

  TableWriter tw;
  Launch sy[SYRK_PATHS][2], rm[2], rt[2];
  for (int w = 0; w < 2; ++w) {
    sy[P_DENSE][w] = fill_syrk<DenseKM>(tw, gp, gp.members[P_DENSE][w], jobs, partials, copies);
    sy[P_CONVG][w] = fill_syrk<ConvG>(tw, gp, gp.members[P_CONVG][w], jobs, partials, copies);
    sy[P_CONVA][w] = fill_syrk<ConvA>(tw, gp, gp.members[P_CONVA][w], jobs, partials, copies);
    sy[P_CONVP][w] = fill_syrk<ConvP>(tw, gp, gp.members[P_CONVP][w], jobs, partials, copies);
    rm[w] = fill_reduce(tw, gp, gp.reduce_many[w], jobs, partials, true);
    rt[w] = fill_reduce(tw, gp, gp.reduce_tile[w], jobs, partials, false);
  }
  const Launch pl = fill_planes(tw, gp, jobs, copies);
  if (tw.words.size() * 4 > gp.table_bytes) return KFAC_ERR_LAUNCH;     // (cannot happen)
  upload_table(tw.words.data(), tw.words.size() * 4, table, stream);
  if (pl.njobs)
    hipLaunchKernelGGL(conv_planes_kernel, dim3(pl.items), dim3(256), 0, stream,
                       (const PlaneJob*)(table + pl.jobs_off), (const int*)(table + pl.cum_off),
                       pl.njobs);
  for (int i : gp.singles) {
    const int st = run_single(jobs[i], gp.single_bytes ? single_ws : nullptr, gp.single_bytes,
                              stream_);
    if (st != KFAC_OK) return st;
  }
  if (!gp.taps.empty()) {
    const std::vector<TapsJob> tj = taps_jobs(gp, jobs);
    const int st = conv_a_taps_grouped((int)tj.size(), tj.data(), taps_ws, gp.taps_bytes, stream);
    if (st != KFAC_OK) return st;
  }
  bool ok = true;
  ok = ok && launch_syrk_group<ConvP, 2>(sy[P_CONVP][1], table, stream);
  ok = ok && launch_syrk_group<ConvA, 2>(sy[P_CONVA][1], table, stream);
  ok = ok && launch_syrk_group<ConvG, 2>(sy[P_CONVG][1], table, stream);
  ok = ok && launch_syrk_group<DenseKM, 2>(sy[P_DENSE][1], table, stream);
  ok = ok && launch_syrk_group<ConvP, 1>(sy[P_CONVP][0], table, stream);
  ok = ok && launch_syrk_group<ConvA, 1>(sy[P_CONVA][0], table, stream);
  ok = ok && launch_syrk_group<ConvG, 1>(sy[P_CONVG][0], table, stream);
  ok = ok && launch_syrk_group<DenseKM, 1>(sy[P_DENSE][0], table, stream);
  if (!ok) return KFAC_ERR_LAUNCH;
  if (rm[1].njobs)
    hipLaunchKernelGGL(reduce_many_grouped_kernel<128>, dim3(rm[1].items), dim3(256), 0, stream,
                       (const RdJob*)(table + rm[1].jobs_off), (const int*)(table + rm[1].cum_off),
                       rm[1].njobs);
  if (rt[1].njobs)
    hipLaunchKernelGGL(reduce_tile_grouped_kernel<128>, dim3(rt[1].items), dim3(256), 0, stream,
                       (const RdJob*)(table + rt[1].jobs_off), (const int*)(table + rt[1].cum_off),
                       rt[1].njobs);
  if (rm[0].njobs)
    hipLaunchKernelGGL(reduce_many_grouped_kernel<64>, dim3(rm[0].items), dim3(256), 0, stream,
                       (const RdJob*)(table + rm[0].jobs_off), (const int*)(table + rm[0].cum_off),
                       rm[0].njobs);
  if (rt[0].njobs)
    hipLaunchKernelGGL(reduce_tile_grouped_kernel<64>, dim3(rt[0].items), dim3(256), 0, stream,
                       (const RdJob*)(table + rt[0].jobs_off), (const int*)(table + rt[0].cum_off),
                       rt[0].njobs);
  return launch_status();
}

}  // extern "C"
