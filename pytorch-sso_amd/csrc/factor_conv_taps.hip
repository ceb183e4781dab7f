// A factor of a stride-1 Conv2d by spatial correlations.
//
// With M = im2col(x), the block of A = M M^T that couples kernel tap t = (kh, kw)
// with tap t' = (kh', kw') is
//     A[(c,t),(c',t')] = sum_{n,oh,ow} x~[n,c,oh+oy_t,ow+ox_t] * x~[n,c',oh+oy_t',ow+ox_t']
// (x~ = zero-padded input, o = tap*dilation - padding).  For stride 1 this is the
// spatial cross-correlation of channel c with channel c' at displacement
// delta = o_t' - o_t, summed over a rectangular window of positions that depends
// on (t, t') only through a few boundary rows and columns.  All blocks with the
// same displacement therefore share one product over the interior, and differ by
// thin edge strips.  For a 3x3 kernel the 45 block products of the upper triangle
// collapse to 13 interior products (one per displacement of the half plane) plus
// strips of one row or column: about 3.4x fewer flops than the im2col product,
// with no bounds check anywhere (every piece lies inside the image).
//
//  1. host: per axis, the windows of all tap pairs are cut into disjoint pieces
//     (plan_axis); a job = (displacement, piece_y, piece_x);
//  2. corr_kernel: R_job[c][c'] = sum over the job's rectangle, on the MFMA tile
//     engine, k-split across workgroups, partial sums into the workspace;
//  3. block_sum_kernel: B[(t,t')][c][c'] = sum over the block's jobs and their
//     k-splits, in a fixed order (t <= t');
//  4. interleave_kernel: A[(c,t),(c',t')] = alpha * B + beta * A_old, with the
//     blocks below the diagonal taken transposed; the elements pass through LDS so
//     that both the reads of B and the writes of A are row-contiguous.
#include <limits.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "common.h"
#include "operands.h"

namespace kfac {

// x[n][c][u0 + ry + dy][v0 + rx + dx] for k = (n, ry, rx) inside a hh x ww rectangle
struct ShiftX {
  static constexpr int layout = MK;
  static constexpr bool has_second = false;
  const float* p;
  int C, H, W, u0, v0, hh, ww;     // u0, v0 already include the displacement
  FastDiv by_area, by_ww;
  struct MS { unsigned off; };
  struct KS { unsigned off; };
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const { return make_rsrc(p); }
  __device__ __forceinline__ MS mstate(int m) const {
    return MS{m < C ? (unsigned)(m * H * W) * 4u : INV_M};
  }
  __device__ __forceinline__ KS kstate(int k, bool valid) const {
    const int n = by_area.div(k);
    const int rem = k - n * hh * ww;
    const int ry = by_ww.div(rem);
    const int rx = rem - ry * ww;
    return KS{k_offset_or_invalid((unsigned)(n * C * H * W + (u0 + ry) * W + v0 + rx) * 4u, valid)};
  }
  __device__ __forceinline__ unsigned off(const MS& m, const KS& k) const { return m.off + k.off; }
  __device__ __forceinline__ bool is_one(const MS&) const { return false; }
};

struct JobDesc {
  short u0, v0, hh, ww;    // rectangle of the first factor; the reduction runs over n * hh * ww
  short dy, dx;            // displacement of the second factor
  short splits;            // k-splits
  unsigned char sh_area, sh_ww;   // shifts of the two FastDiv (by hh * ww and by ww)
  unsigned m_area, m_ww;          // their multipliers
  int cps;                 // chunks per split
  int part0;               // index (in C*C units) of its first partial in the workspace
};

constexpr int MAX_JOBS = 64;
constexpr int MAX_TAPS = 9;
constexpr int MAX_PAIRS = MAX_TAPS * (MAX_TAPS + 1) / 2;
constexpr int MAX_PAIR_JOBS = 512;     // pool shared by all pairs
constexpr int IL_ROWS = 16;            // interleave_kernel: channels per workgroup along the rows
constexpr int IL_COLS = 32;            //                    and along the columns of A

// The whole plan travels as a kernel argument (below the 4 KiB limit).
struct TapPlanDev {
  JobDesc jobs[MAX_JOBS];
  int item0[MAX_JOBS];     // first work item of each job; INT_MAX past the last job
  int njobs;
  int npairs;
  unsigned char pair_t[MAX_PAIRS + 3];       // t * 16 + t'
  unsigned char pair_of[MAX_TAPS * MAX_TAPS + 3];   // [t * T + t'] -> pair (t <= t')
  short pair_first[MAX_PAIRS + 1];           // into pair_jobs
  short pair_jobs[MAX_PAIR_JOBS];
};
static_assert(sizeof(TapPlanDev) <= 3800, "plan must fit the kernel argument buffer");
// the product of one work item: tile `tile` of job j over its k-split `split`
template <int W>
__device__ __forceinline__ void corr_product(const float* x, int nimg, int C, int H, int Wd,
                                             const TapPlanDev& plan, int tiles_side, float* ws,
                                             int j, int split, int tile, float* smem) {
  constexpr int TS = 64 * W;
  constexpr int KC = Cfg<W, W>::KC;
  const JobDesc jd = plan.jobs[j];
  const int bi = tile / tiles_side, bj = tile - bi * tiles_side;
  const int K = nimg * jd.hh * jd.ww;
  const int kbeg = split * jd.cps * KC;
  int kend = kbeg + jd.cps * KC;
  if (kend > K) kend = K;
  FastDiv by_area, by_ww;
  by_area.m = jd.m_area;
  by_area.sh = jd.sh_area;
  by_ww.m = jd.m_ww;
  by_ww.sh = jd.sh_ww;
  ShiftX P{x, C, H, Wd, jd.u0, jd.v0, jd.hh, jd.ww, by_area, by_ww};
  ShiftX Q{x, C, H, Wd, jd.u0 + jd.dy, jd.v0 + jd.dx, jd.hh, jd.ww, by_area, by_ww};
  EpiStore epi{ws + (size_t)(jd.part0 + split) * C * C, C, C, C, 1.f, 0.f, false};
  gemm_tile_cfg<W, W>(P, Q, bi * TS, bj * TS, kbeg, kend, false, epi, smem);
}

// work item `item` of one layer's plan -> (job, split, tile), job by job
template <int W>
__device__ __forceinline__ void corr_item(const float* x, int nimg, int C, int H, int Wd,
                                          const TapPlanDev& plan, int tiles_side, float* ws,
                                          int item, float* smem) {
  int j = -1;
#pragma unroll
  for (int q = 0; q < MAX_JOBS; ++q) j += plan.item0[q] <= item ? 1 : 0;
  const int ntiles = tiles_side * tiles_side;
  const int local = item - plan.item0[j];
  const int split = local / ntiles;
  corr_product<W>(x, nimg, C, H, Wd, plan, tiles_side, ws, j, split, local - split * ntiles, smem);
}

template <int W>
__global__ __launch_bounds__(64 * W * W, W == 2 ? 3 : 1) void corr_kernel(
    const float* x, int nimg, int C, int H, int Wd, const TapPlanDev plan, int tiles_side,
    float* ws) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  corr_item<W>(x, nimg, C, H, Wd, plan, tiles_side, ws, blockIdx.x, smem);
}

// The items of a layer in the order of a grouped launch, as a table of (job, k-split)
// entries (tile fastest within an entry).  The jobs with many splits (the interior
// products, one per displacement) come first, k-split by k-split: a run of consecutive
// entries then reads one region of the input under all displacements, and
// xcd_remap_range gives every XCD such a run, so that the region is fetched into one L2
// once (job by job, the whole input streams through every L2 once per displacement).  The
// short jobs (edge strips) follow job by job and are dealt round-robin: a launch of this
// kind is resident all at once, a compute unit holds 5 or 6 of its items, and the units
// with one more should get a short one.
struct TapOrder {
  int first;            // of this layer's entries in the table
  int main_items;       // items (entries x tiles) that are remapped per XCD
};
__host__ __device__ __forceinline__ unsigned order_entry(int job, int split) {
  return (unsigned)job | ((unsigned)split << 8);
}

// One layer of a grouped call: its tensors, and where its plan's partials and block sums live.
struct TapLayer {
  const float* x;
  float* ws;
  float* B;
  const float* Ain;
  float* A;
  int n, C, H, W, T, tiles_side;
  float alpha, beta;
};

__device__ __forceinline__ int find_layer(const int* __restrict__ cum, int n, int item) {
  int lo = 0, hi = n;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cum[mid] <= item) lo = mid; else hi = mid;
  }
  return lo;
}

// the correlation items of all layers of one tile size in one launch
template <int W>
__global__ __launch_bounds__(64 * W * W, W == 2 ? 3 : 1) void corr_grouped_kernel(
    const TapLayer* __restrict__ layers, const TapPlanDev* __restrict__ plans,
    const TapOrder* __restrict__ order, const unsigned* __restrict__ entries,
    const int* __restrict__ index, const int* __restrict__ cum, int nlayers) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int k = find_layer(cum, nlayers, blockIdx.x);
  const int l = index[k];
  const TapLayer& L = layers[l];
  const TapOrder o = order[l];
  int v = blockIdx.x - cum[k];
  if (v < o.main_items) v = xcd_remap_range(blockIdx.x, cum[k], o.main_items);
  const int ntiles = L.tiles_side * L.tiles_side;
  const int e = v / ntiles;
  const unsigned entry = entries[o.first + e];
  corr_product<W>(L.x, L.n, L.C, L.H, L.W, plans[l], L.tiles_side, L.ws, (int)(entry & 255u),
                  (int)(entry >> 8), v - e * ntiles, smem);
}

// B[pair][c][c'] = sum over the pair's jobs and their k-splits, in a fixed order.
// One workgroup owns 64 float4 groups of the block; its 4 waves take the partials
// (all splits of all jobs, as one list) round-robin, two loads in flight each, and
// the 4 wave sums are added in wave order.
__device__ __forceinline__ void block_sum_item(const TapPlanDev& plan, const float* ws, int CC,
                                               float* B, int eblock, int pair) {
  __shared__ float4 red[4][64];
  const int jb = plan.pair_first[pair], je = plan.pair_first[pair + 1];
  const int lane = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int e = (eblock * 64 + lane) * 4;   // CC is a multiple of 4 (channel counts are even, >= 16)
  const bool live = e < CC;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  int turn = 0;                                 // position in the pair's list of partials, mod 4
  if (live) {
    for (int q = jb; q < je; ++q) {
      const JobDesc jd = plan.jobs[plan.pair_jobs[q]];
      const float* part = ws + (size_t)jd.part0 * CC + e;
      int sp = (sl - turn) & 3;                 // first split of this job that is this wave's turn
      for (; sp + 4 < jd.splits; sp += 8) {
        const float4 v0 = *reinterpret_cast<const float4*>(part + (size_t)sp * CC);
        const float4 v1 = *reinterpret_cast<const float4*>(part + (size_t)(sp + 4) * CC);
        s.x += v0.x; s.y += v0.y; s.z += v0.z; s.w += v0.w;
        s.x += v1.x; s.y += v1.y; s.z += v1.z; s.w += v1.w;
      }
      if (sp < jd.splits) {
        const float4 v = *reinterpret_cast<const float4*>(part + (size_t)sp * CC);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
      }
      turn = (turn + jd.splits) & 3;
    }
  }
  red[sl][lane] = s;
  __syncthreads();
  if (sl == 0 && live) {
    float4 t = red[0][lane];
#pragma unroll
    for (int k = 1; k < 4; ++k) {
      const float4 v = red[k][lane];
      t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
    }
    *reinterpret_cast<float4*>(B + (size_t)pair * CC + e) = t;
  }
}

__global__ __launch_bounds__(256) void block_sum_kernel(const TapPlanDev plan, const float* ws,
                                                        int CC, float* B) {
  block_sum_item(plan, ws, CC, B, blockIdx.x, blockIdx.y);
}

// ... of all layers: item = (layer, pair, block of 1024 elements).  A grouped plan cuts the
// jobs into few, long splits, so a pair's list of partials is short: every thread owns one
// float4 of the block and walks the whole list itself (fixed order, four loads in flight)
// instead of four waves sharing the list of a quarter as many elements.
constexpr int SUM_BLOCK = 1024;
__global__ __launch_bounds__(256) void block_sum_grouped_kernel(
    const TapLayer* __restrict__ layers, const TapPlanDev* __restrict__ plans,
    const int* __restrict__ cum, int nlayers) {
  const int l = find_layer(cum, nlayers, blockIdx.x);
  const TapLayer& L = layers[l];
  const TapPlanDev& plan = plans[l];
  const int CC = L.C * L.C;
  const int eblocks = (CC + SUM_BLOCK - 1) / SUM_BLOCK;
  const int local = blockIdx.x - cum[l];
  const int pair = local / eblocks;
  const int e = ((local - pair * eblocks) * 256 + threadIdx.x) * 4;
  if (e >= CC) return;
  const int jb = plan.pair_first[pair], je = plan.pair_first[pair + 1];
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int q = jb; q < je; ++q) {
    const JobDesc& jd = plan.jobs[plan.pair_jobs[q]];
    const float* part = L.ws + (size_t)jd.part0 * CC + e;
    const int splits = jd.splits;
    int sp = 0;
    for (; sp + 4 <= splits; sp += 4) {
      const float4 v0 = *reinterpret_cast<const float4*>(part + (size_t)sp * CC);
      const float4 v1 = *reinterpret_cast<const float4*>(part + (size_t)(sp + 1) * CC);
      const float4 v2 = *reinterpret_cast<const float4*>(part + (size_t)(sp + 2) * CC);
      const float4 v3 = *reinterpret_cast<const float4*>(part + (size_t)(sp + 3) * CC);
      s.x += v0.x; s.y += v0.y; s.z += v0.z; s.w += v0.w;
      s.x += v1.x; s.y += v1.y; s.z += v1.z; s.w += v1.w;
      s.x += v2.x; s.y += v2.y; s.z += v2.z; s.w += v2.w;
      s.x += v3.x; s.y += v3.y; s.z += v3.z; s.w += v3.w;
    }
    for (; sp < splits; ++sp) {
      const float4 v = *reinterpret_cast<const float4*>(part + (size_t)sp * CC);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  }
  *reinterpret_cast<float4*>(L.B + (size_t)pair * CC + e) = s;
}

// One workgroup writes, for one tap t, the rows (c, t) of 16 channels c against the
// columns (c', t') of 32 channels c' and all taps t': 16 runs of 32*T consecutive
// elements of A.  The T blocks B[(t,t')] that feed them are read along their rows
// (blocks below the diagonal: the transposed block, along its rows as well) and
// go through LDS into the interleaved order.
__device__ __forceinline__ void interleave_item(const TapPlanDev& plan, const float* B, int C,
                                                int T, float alpha, float beta, const float* Ain,
                                                float* A, int qblock, int cblock, int t) {
  __shared__ float out[IL_ROWS][IL_COLS * MAX_TAPS + 1];
  const int c0 = cblock * IL_ROWS, q0 = qblock * IL_COLS;
  const int d = C * T;
  const size_t CC = (size_t)C * C;
  const int tid = threadIdx.x;
  for (int t2 = 0; t2 < T; ++t2) {
    if (t <= t2) {
      // B[(t,t2)][c][c2]: lanes along c2
      const float* blk = B + plan.pair_of[t * T + t2] * CC;
      const int j = tid % IL_COLS;
#pragma unroll
      for (int k = 0; k < IL_ROWS * IL_COLS / 256; ++k) {
        const int i = tid / IL_COLS + (256 / IL_COLS) * k;
        const int c = c0 + i, c2 = q0 + j;
        out[i][j * T + t2] = (c < C && c2 < C) ? blk[(size_t)c * C + c2] : 0.f;
      }
    } else {
      // transposed block B[(t2,t)][c2][c]: lanes along c
      const float* blk = B + plan.pair_of[t2 * T + t] * CC;
      const int i = tid % IL_ROWS;
#pragma unroll
      for (int k = 0; k < IL_ROWS * IL_COLS / 256; ++k) {
        const int j = tid / IL_ROWS + (256 / IL_ROWS) * k;
        const int c = c0 + i, c2 = q0 + j;
        out[i][j * T + t2] = (c < C && c2 < C) ? blk[(size_t)c2 * C + c] : 0.f;
      }
    }
  }
  __syncthreads();
  const int ncols = min(IL_COLS, C - q0) * T;       // run length in A
  const int nrows = min(IL_ROWS, C - c0);
  const int total = nrows * ncols;
  const float* prev = Ain ? Ain : A;
  constexpr int BATCH = 6;
  for (int e0 = tid; e0 < total; e0 += 256 * BATCH) {
    float old[BATCH];
    size_t idx[BATCH];
    float val[BATCH];
#pragma unroll
    for (int k = 0; k < BATCH; ++k) {
      const int e = e0 + 256 * k;
      const int i = e / ncols, q = e - i * ncols;
      const bool in = e < total;
      idx[k] = in ? (size_t)((c0 + i) * T + t) * d + (size_t)q0 * T + q : 0;
      val[k] = in ? out[i][q] : 0.f;
      old[k] = (in && beta != 0.f) ? prev[idx[k]] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < BATCH; ++k)
      if (e0 + 256 * k < total) A[idx[k]] = alpha * val[k] + beta * old[k];
  }
}

__global__ __launch_bounds__(256) void interleave_kernel(const TapPlanDev plan, const float* B,
                                                         int C, int T, float alpha, float beta,
                                                         const float* Ain, float* A) {
  interleave_item(plan, B, C, T, alpha, beta, Ain, A, blockIdx.x, blockIdx.y, blockIdx.z);
}

// ... of all layers: item = (layer, tap, block of 16 channels, block of 32 channels)
__global__ __launch_bounds__(256) void interleave_grouped_kernel(
    const TapLayer* __restrict__ layers, const TapPlanDev* __restrict__ plans,
    const int* __restrict__ cum, int nlayers) {
  const int l = find_layer(cum, nlayers, blockIdx.x);
  const TapLayer& L = layers[l];
  const int qb = (L.C + IL_COLS - 1) / IL_COLS, cb = (L.C + IL_ROWS - 1) / IL_ROWS;
  int local = blockIdx.x - cum[l];
  const int t = local / (qb * cb);
  local -= t * qb * cb;
  const int cblock = local / qb;
  interleave_item(plans[l], L.B, L.C, L.T, L.alpha, L.beta, L.Ain, L.A, local - cblock * qb,
                  cblock, t);
}

// ---------------------------------------------------------------------------
// host-side planning
// ---------------------------------------------------------------------------
struct AxisPiece {
  int delta, lo, hi;      // first-factor coordinates [lo, hi)
};

struct AxisPlan {
  std::vector<AxisPiece> pieces;
  // for tap pair (a, a'): indices of the pieces that make up its window
  std::vector<std::vector<int>> pair_pieces;   // [a * K + a']
};

static AxisPlan plan_axis(int size, int out, int K, int dil, int pad) {
  AxisPlan ap;
  ap.pair_pieces.resize((size_t)K * K);
  struct Win { int a, b, delta, lo, hi; };
  std::vector<Win> wins;
  for (int a = 0; a < K; ++a)
    for (int b = 0; b < K; ++b) {
      const int oa = a * dil - pad, ob = b * dil - pad;
      const int lo = std::max(0, std::max(-oa, -ob));
      const int hi = std::min(out, std::min(size - oa, size - ob));
      if (hi > lo) wins.push_back(Win{a, b, ob - oa, lo + oa, hi + oa});
    }
  // per displacement: cut at every window boundary
  std::vector<int> deltas;
  for (auto& w : wins) deltas.push_back(w.delta);
  std::sort(deltas.begin(), deltas.end());
  deltas.erase(std::unique(deltas.begin(), deltas.end()), deltas.end());
  for (int dl : deltas) {
    std::vector<int> cuts;
    for (auto& w : wins)
      if (w.delta == dl) { cuts.push_back(w.lo); cuts.push_back(w.hi); }
    std::sort(cuts.begin(), cuts.end());
    cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
    for (size_t i = 0; i + 1 < cuts.size(); ++i) {
      const int lo = cuts[i], hi = cuts[i + 1];
      std::vector<const Win*> users;
      for (auto& w : wins)
        if (w.delta == dl && w.lo <= lo && hi <= w.hi) users.push_back(&w);
      if (users.empty()) continue;
      const int idx = (int)ap.pieces.size();
      ap.pieces.push_back(AxisPiece{dl, lo, hi});
      for (auto* w : users) ap.pair_pieces[(size_t)w->a * K + w->b].push_back(idx);
    }
  }
  return ap;
}

struct TapPlanHost {
  TapPlanDev dev;
  int tiles_side, w, items;
  size_t partial_floats, sum_offset;
  bool ok;
};

// `group_cps` > 0: the plan is for a launch shared with other layers, which fills the chip
// whatever this layer contributes: every job is then cut into items of about that many
// chunks (fewer, longer items: fewer partial blocks to write and to add up).
static TapPlanHost plan_taps(int n, int c, int H, int Wd, int kh, int kw, int ph, int pw, int dh,
                             int dw, int group_cps = 0) {
  TapPlanHost hp;
  hp.ok = false;
  const int T = kh * kw;
  if (T < 2 || T > MAX_TAPS) return hp;
  const int OH = H + 2 * ph - dh * (kh - 1), OW = Wd + 2 * pw - dw * (kw - 1);
  if (OH <= 0 || OW <= 0) return hp;
  const AxisPlan ay = plan_axis(H, OH, kh, dh, ph), ax = plan_axis(Wd, OW, kw, dw, pw);
  TapPlanDev& pd = hp.dev;
  memset(&pd, 0, sizeof(pd));
  std::vector<long> job_key;
  int npj = 0;
  pd.pair_first[0] = 0;
  for (int t = 0; t < T; ++t)
    for (int t2 = t; t2 < T; ++t2) {
      const int a = t / kw, b = t % kw, a2 = t2 / kw, b2 = t2 % kw;
      pd.pair_t[pd.npairs] = (unsigned char)(t * 16 + t2);
      pd.pair_of[t * T + t2] = (unsigned char)pd.npairs;
      for (int py : ay.pair_pieces[(size_t)a * kh + a2])
        for (int px : ax.pair_pieces[(size_t)b * kw + b2]) {
          const long key = (long)py * 4096 + px;
          int j = 0;
          while (j < (int)job_key.size() && job_key[j] != key) ++j;
          if (j == (int)job_key.size()) {
            if (pd.njobs >= MAX_JOBS) return hp;
            job_key.push_back(key);
            JobDesc& jd = pd.jobs[pd.njobs++];
            jd.u0 = (short)ay.pieces[py].lo;
            jd.hh = (short)(ay.pieces[py].hi - ay.pieces[py].lo);
            jd.dy = (short)ay.pieces[py].delta;
            jd.v0 = (short)ax.pieces[px].lo;
            jd.ww = (short)(ax.pieces[px].hi - ax.pieces[px].lo);
            jd.dx = (short)ax.pieces[px].delta;
            const FastDiv fa((unsigned)(jd.hh * jd.ww)), fw((unsigned)jd.ww);
            jd.m_area = fa.m;
            jd.sh_area = (unsigned char)fa.sh;
            jd.m_ww = fw.m;
            jd.sh_ww = (unsigned char)fw.sh;
          }
          if (npj >= MAX_PAIR_JOBS) return hp;
          pd.pair_jobs[npj++] = (short)j;
        }
      ++pd.npairs;
      pd.pair_first[pd.npairs] = (short)npj;
    }
  // tiles and k-splits: work items in proportion to each job's length
  hp.w = c <= 64 ? 1 : 2;
  const int ts = 64 * hp.w;
  hp.tiles_side = cdiv(c, ts);
  const int ntiles = hp.tiles_side * hp.tiles_side;
  const int kc = hp.w == 1 ? Cfg<1, 1>::KC : Cfg<2, 2>::KC;
  double total = 0;
  auto job_k = [&](const JobDesc& jd) { return (long)n * jd.hh * jd.ww; };
  for (int j = 0; j < pd.njobs; ++j) total += (double)job_k(pd.jobs[j]);
  // All workgroups of a launch that fits the chip are resident at once (3 four-wave
  // workgroups per CU: 768) and share the matrix cores of their CU, so the launch lasts as
  // long as the fullest CU: a little under one full round (the split counts round up) beats
  // 1.3 rounds by a quarter.  The one-wave workgroups (8 per CU) do best at 1.5 rounds.
  const double target_items = hp.w == 1 ? 3072.0 : 700.0;
  int item = 0, part = 0;
  for (int j = 0; j < pd.njobs; ++j) {
    JobDesc& jd = pd.jobs[j];
    const long nchunks = (job_k(jd) + kc - 1) / kc;
    long splits = group_cps > 0
                      ? (nchunks + group_cps / 2) / group_cps
                      : (long)(target_items * ((double)job_k(jd) / total) / ntiles + 0.5);
    const long max_splits = std::max<long>(1, nchunks / (128 / kc));
    splits = std::max<long>(1, std::min(std::min(splits, max_splits), 4096L));
    long cps = (nchunks + splits - 1) / splits;
    splits = (nchunks + cps - 1) / cps;
    jd.splits = (short)splits;
    jd.cps = (int)cps;
    pd.item0[j] = item;
    jd.part0 = part;
    item += (int)splits * ntiles;
    part += (int)splits;
  }
  for (int j = pd.njobs; j < MAX_JOBS; ++j) pd.item0[j] = INT_MAX;
  hp.items = item;
  hp.partial_floats = (size_t)(part + pd.npairs) * c * c;     // partials, then the block sums
  hp.sum_offset = (size_t)part * c * c;
  hp.ok = true;
  return hp;
}

bool conv_a_taps_applicable(int c, int kh, int kw, int sh, int sw, int add_bias) {
  return sh == 1 && sw == 1 && !add_bias && kh * kw >= 2 && kh * kw <= MAX_TAPS && c >= 16 &&
         c % 2 == 0;
}

size_t conv_a_taps_workspace(int n, int c, int H, int W, int kh, int kw, int ph, int pw, int dh,
                             int dw) {
  const TapPlanHost hp = plan_taps(n, c, H, W, kh, kw, ph, pw, dh, dw);
  return hp.ok ? hp.partial_floats * sizeof(float) : 0;
}

// MFMA flops corr_kernel executes for this geometry: whole chunks on full tiles, for every
// (job, split, tile) work item.
static double plan_executed_flops(const TapPlanHost& hp, int n) {
  const int ts = 64 * hp.w;
  const int kc = hp.w == 1 ? Cfg<1, 1>::KC : Cfg<2, 2>::KC;
  const double ntiles = (double)hp.tiles_side * hp.tiles_side;
  double total = 0.;
  for (int j = 0; j < hp.dev.njobs; ++j) {
    const JobDesc& jd = hp.dev.jobs[j];
    const long K = (long)n * jd.hh * jd.ww;
    total += ntiles * (double)((K + kc - 1) / kc) * kc * 2.0 * ts * ts;
  }
  return total;
}

double conv_a_taps_executed_flops(int n, int c, int H, int W, int kh, int kw, int ph, int pw,
                                  int dh, int dw) {
  const TapPlanHost hp = plan_taps(n, c, H, W, kh, kw, ph, pw, dh, dw);
  return hp.ok ? plan_executed_flops(hp, n) : 0.;
}

// returns KFAC_OK, an error, or -1 when the geometry is not covered (the caller
// then uses the im2col kernel)
int conv_a_taps(const float* x, int n, int c, int H, int W, int kh, int kw, int ph, int pw, int dh,
                int dw, float alpha, float beta, const float* A_prev, float* A, void* workspace,
                size_t workspace_bytes, hipStream_t stream) {
  const TapPlanHost hp = plan_taps(n, c, H, W, kh, kw, ph, pw, dh, dw);
  if (!hp.ok) return -1;
  if (!workspace || workspace_bytes < hp.partial_floats * sizeof(float)) return KFAC_ERR_WORKSPACE;
  float* ws = (float*)workspace;
  float* B = ws + hp.sum_offset;
  const int T = kh * kw;
  if (hp.w == 1) {
    constexpr int lds = Cfg<1, 1>::SMEM_FLOATS * (int)sizeof(float);
    if (!enable_large_lds((const void*)corr_kernel<1>, lds)) return KFAC_ERR_LAUNCH;
    hipLaunchKernelGGL(corr_kernel<1>, dim3(hp.items), dim3(64), lds, stream, x, n, c, H, W,
                       hp.dev, hp.tiles_side, ws);
  } else {
    constexpr int lds = Cfg<2, 2>::SMEM_FLOATS * (int)sizeof(float);
    if (!enable_large_lds((const void*)corr_kernel<2>, lds)) return KFAC_ERR_LAUNCH;
    hipLaunchKernelGGL(corr_kernel<2>, dim3(hp.items), dim3(256), lds, stream, x, n, c, H, W,
                       hp.dev, hp.tiles_side, ws);
  }
  hipLaunchKernelGGL(block_sum_kernel, dim3(cdiv(c * c / 4, 64), hp.dev.npairs), dim3(256), 0,
                     stream, hp.dev, ws, c * c, B);
  hipLaunchKernelGGL(interleave_kernel, dim3(cdiv(c, IL_COLS), cdiv(c, IL_ROWS), T), dim3(256), 0,
                     stream, hp.dev, B, c,
                     T, alpha, beta, A_prev, A);
  return launch_status();
}

// ---------------------------------------------------------------------------
// several layers at once
// ---------------------------------------------------------------------------
struct TapsShape {
  int n, c, H, W, kh, kw, ph, pw, dh, dw;
  bool operator==(const TapsShape& o) const { return memcmp(this, &o, sizeof(TapsShape)) == 0; }
};

// Everything of a grouped call that depends on the shapes only.
struct TapsGroupPlan {
  std::vector<TapsShape> shapes;
  std::vector<TapPlanHost> plans;
  std::vector<TapOrder> orders;
  std::vector<unsigned> entries;
  std::vector<size_t> ws_off;          // floats, per layer, from the partial area
  std::vector<int> members[2];         // layers by tile size (w - 1), longest items first
  std::vector<int> cum_corr[2], cum_sum, cum_il;
  size_t layers_off, plans_off, orders_off, entries_off, index_off[2], cum_corr_off[2], cum_sum_off, cum_il_off;
  size_t table_bytes, partial_floats;
  double executed_flops;
  bool ok;
};

static size_t pad16(size_t v) { return (v + 15) / 16 * 16; }

// appends the layer's entries to `entries`; the interior products are the jobs at least
// half as long as the longest
static TapOrder make_order(const TapPlanHost& hp, std::vector<unsigned>& entries) {
  TapOrder o;
  o.first = (int)entries.size();
  const TapPlanDev& pd = hp.dev;
  const int J = pd.njobs, ntiles = hp.tiles_side * hp.tiles_side;
  long longest = 0;
  for (int j = 0; j < J; ++j) longest = std::max(longest, (long)pd.jobs[j].splits * pd.jobs[j].cps);
  auto interior = [&](int j) { return 2L * pd.jobs[j].splits * pd.jobs[j].cps >= longest; };
  int smax = 0;
  for (int j = 0; j < J; ++j)
    if (interior(j)) smax = std::max(smax, (int)pd.jobs[j].splits);
  for (int s = 0; s < smax; ++s)
    for (int j = 0; j < J; ++j)
      if (interior(j) && s < pd.jobs[j].splits) entries.push_back(order_entry(j, s));
  o.main_items = ((int)entries.size() - o.first) * ntiles;
  for (int j = 0; j < J; ++j)
    if (!interior(j))
      for (int s = 0; s < pd.jobs[j].splits; ++s) entries.push_back(order_entry(j, s));
  return o;
}

// chunks per item of a grouped launch (one-wave 64-wide tiles / four-wave 128-wide tiles);
// measured flat between 48 and 192
constexpr int TAPS_GROUP_CPS1 = 192, TAPS_GROUP_CPS2 = 96;

static TapsGroupPlan* make_taps_group_plan(int count, const TapsJob* jobs) {
  TapsGroupPlan* gp = new TapsGroupPlan();
  gp->ok = true;
  gp->partial_floats = 0;
  gp->executed_flops = 0.;
  // chunks per item: the default where a tile size has plenty of work, shorter items where
  // its launch would not fill the chip twice (3 layers of 64 channels, say)
  double units[2] = {0., 0.};
  for (int i = 0; i < count; ++i) {
    const TapsJob& j = jobs[i];
    const int w = j.c <= 64 ? 1 : 2;
    const double tiles = (double)cdiv(j.c, 64 * w) * cdiv(j.c, 64 * w);
    // 13 of the 45 tap pairs of a 3x3 kernel are computed; in general about T(T+1)/2 / 3.4
    const int T = j.kh * j.kw;
    units[w - 1] += tiles * (T * (T + 1) / 2 / 3.4) * ((double)j.n * j.H * j.W / 16.);
  }
  int group_cps[2];
  for (int w = 0; w < 2; ++w) {
    const double slots = w == 0 ? 2048. : 768.;
    const int dflt = w == 0 ? TAPS_GROUP_CPS1 : TAPS_GROUP_CPS2;
    long t = (long)(units[w] / (2. * slots));
    group_cps[w] = (int)std::max(8L, std::min((long)dflt, t));
  }
  for (int i = 0; i < count; ++i) {
    const TapsJob& j = jobs[i];
    gp->shapes.push_back(TapsShape{j.n, j.c, j.H, j.W, j.kh, j.kw, j.ph, j.pw, j.dh, j.dw});
    gp->plans.push_back(plan_taps(j.n, j.c, j.H, j.W, j.kh, j.kw, j.ph, j.pw, j.dh, j.dw,
                                  group_cps[j.c <= 64 ? 0 : 1]));
    const TapPlanHost& hp = gp->plans.back();
    if (!hp.ok) {
      gp->ok = false;
      return gp;
    }
    gp->orders.push_back(make_order(hp, gp->entries));
    gp->ws_off.push_back(gp->partial_floats);
    gp->partial_floats += (hp.partial_floats + 63) / 64 * 64;
    gp->members[hp.w - 1].push_back(i);
    gp->executed_flops += plan_executed_flops(hp, j.n);
  }
  for (int w = 0; w < 2; ++w) {
    auto& m = gp->members[w];
    auto longest = [&](int i) {
      int c = 0;
      for (int q = 0; q < gp->plans[i].dev.njobs; ++q) c = std::max(c, gp->plans[i].dev.jobs[q].cps);
      return c;
    };
    std::stable_sort(m.begin(), m.end(), [&](int a, int b) { return longest(a) > longest(b); });
    int items = 0;
    for (int i : m) {
      gp->cum_corr[w].push_back(items);
      items += gp->plans[i].items;
    }
    gp->cum_corr[w].push_back(items);
  }
  int s_items = 0, il_items = 0;
  for (int i = 0; i < count; ++i) {
    const TapsJob& j = jobs[i];
    const int T = j.kh * j.kw;
    gp->cum_sum.push_back(s_items);
    gp->cum_il.push_back(il_items);
    s_items += cdiv(j.c * j.c, SUM_BLOCK) * gp->plans[i].dev.npairs;
    il_items += cdiv(j.c, IL_COLS) * cdiv(j.c, IL_ROWS) * T;
  }
  gp->cum_sum.push_back(s_items);
  gp->cum_il.push_back(il_items);
  size_t off = 0;
  gp->layers_off = off;
  off += pad16((size_t)count * sizeof(TapLayer));
  gp->plans_off = off;
  off += pad16((size_t)count * sizeof(TapPlanDev));
  gp->orders_off = off;
  off += pad16((size_t)count * sizeof(TapOrder));
  gp->entries_off = off;
  off += pad16(gp->entries.size() * sizeof(unsigned));
  for (int w = 0; w < 2; ++w) {
    gp->index_off[w] = off;
    off += pad16(gp->members[w].size() * sizeof(int));
    gp->cum_corr_off[w] = off;
    off += pad16(gp->cum_corr[w].size() * sizeof(int));
  }
  gp->cum_sum_off = off;
  off += pad16(gp->cum_sum.size() * sizeof(int));
  gp->cum_il_off = off;
  off += pad16(gp->cum_il.size() * sizeof(int));
  gp->table_bytes = (off + 255) / 256 * 256;
  return gp;
}

// the last plans of every host thread are kept (and never freed: nothing of this library
// has a destructor that could run at process exit)
static const TapsGroupPlan& taps_group_plan(int count, const TapsJob* jobs) {
  constexpr int SLOTS = 16;
  static thread_local TapsGroupPlan** slots = nullptr;
  static thread_local int next_slot = 0;
  if (!slots) slots = new TapsGroupPlan*[SLOTS]();
  for (int k = 0; k < SLOTS; ++k) {
    const TapsGroupPlan* p = slots[k];
    if (!p || (int)p->shapes.size() != count) continue;
    bool same = true;
    for (int i = 0; i < count && same; ++i) {
      const TapsJob& j = jobs[i];
      same = p->shapes[i] == TapsShape{j.n, j.c, j.H, j.W, j.kh, j.kw, j.ph, j.pw, j.dh, j.dw};
    }
    if (same) return *p;
  }
  TapsGroupPlan*& slot = slots[next_slot];
  next_slot = (next_slot + 1) % SLOTS;
  delete slot;
  slot = make_taps_group_plan(count, jobs);
  return *slot;
}

size_t conv_a_taps_grouped_workspace(int count, const TapsJob* jobs) {
  if (count <= 0) return 0;
  const TapsGroupPlan& gp = taps_group_plan(count, jobs);
  return gp.ok ? gp.table_bytes + gp.partial_floats * sizeof(float) : 0;
}

double conv_a_taps_grouped_executed_flops(int count, const TapsJob* jobs) {
  if (count <= 0) return 0.;
  const TapsGroupPlan& gp = taps_group_plan(count, jobs);
  return gp.ok ? gp.executed_flops : 0.;
}

int conv_a_taps_grouped(int count, const TapsJob* jobs, void* workspace, size_t workspace_bytes,
                        hipStream_t stream) {
  if (count <= 0) return KFAC_OK;
  const TapsGroupPlan& gp = taps_group_plan(count, jobs);
  if (!gp.ok) return KFAC_ERR_ARG;
  if (!workspace || workspace_bytes < gp.table_bytes + gp.partial_floats * sizeof(float))
    return KFAC_ERR_WORKSPACE;
  char* table = (char*)workspace;
  float* partials = (float*)(table + gp.table_bytes);
  std::vector<char> img(gp.table_bytes, 0);
  TapLayer* layers = (TapLayer*)(img.data() + gp.layers_off);
  TapPlanDev* plans = (TapPlanDev*)(img.data() + gp.plans_off);
  for (int i = 0; i < count; ++i) {
    const TapsJob& j = jobs[i];
    const TapPlanHost& hp = gp.plans[i];
    float* ws = partials + gp.ws_off[i];
    layers[i] = TapLayer{j.x, ws, ws + hp.sum_offset, j.A_prev, j.A, j.n, j.c, j.H, j.W,
                         j.kh * j.kw, hp.tiles_side, j.alpha, j.beta};
    plans[i] = hp.dev;
  }
  memcpy(img.data() + gp.orders_off, gp.orders.data(), (size_t)count * sizeof(TapOrder));
  memcpy(img.data() + gp.entries_off, gp.entries.data(), gp.entries.size() * sizeof(unsigned));
  for (int w = 0; w < 2; ++w) {
    if (!gp.members[w].empty())
      memcpy(img.data() + gp.index_off[w], gp.members[w].data(), gp.members[w].size() * sizeof(int));
    memcpy(img.data() + gp.cum_corr_off[w], gp.cum_corr[w].data(), gp.cum_corr[w].size() * sizeof(int));
  }
  memcpy(img.data() + gp.cum_sum_off, gp.cum_sum.data(), gp.cum_sum.size() * sizeof(int));
  memcpy(img.data() + gp.cum_il_off, gp.cum_il.data(), gp.cum_il.size() * sizeof(int));
  upload_table(img.data(), img.size(), table, stream);
  const TapLayer* dl = (const TapLayer*)(table + gp.layers_off);
  const TapPlanDev* dp = (const TapPlanDev*)(table + gp.plans_off);
  const TapOrder* dord = (const TapOrder*)(table + gp.orders_off);
  const unsigned* dent = (const unsigned*)(table + gp.entries_off);
  if (!gp.members[1].empty()) {
    constexpr int lds = Cfg<2, 2>::SMEM_FLOATS * (int)sizeof(float);
    if (!enable_large_lds((const void*)corr_grouped_kernel<2>, lds)) return KFAC_ERR_LAUNCH;
    hipLaunchKernelGGL(corr_grouped_kernel<2>, dim3(gp.cum_corr[1].back()), dim3(256), lds, stream,
                       dl, dp, dord, dent, (const int*)(table + gp.index_off[1]),
                       (const int*)(table + gp.cum_corr_off[1]), (int)gp.members[1].size());
  }
  if (!gp.members[0].empty()) {
    constexpr int lds = Cfg<1, 1>::SMEM_FLOATS * (int)sizeof(float);
    if (!enable_large_lds((const void*)corr_grouped_kernel<1>, lds)) return KFAC_ERR_LAUNCH;
    hipLaunchKernelGGL(corr_grouped_kernel<1>, dim3(gp.cum_corr[0].back()), dim3(64), lds, stream,
                       dl, dp, dord, dent, (const int*)(table + gp.index_off[0]),
                       (const int*)(table + gp.cum_corr_off[0]), (int)gp.members[0].size());
  }
  hipLaunchKernelGGL(block_sum_grouped_kernel, dim3(gp.cum_sum.back()), dim3(256), 0, stream, dl, dp,
                     (const int*)(table + gp.cum_sum_off), count);
  hipLaunchKernelGGL(interleave_grouped_kernel, dim3(gp.cum_il.back()), dim3(256), 0, stream, dl, dp,
                     (const int*)(table + gp.cum_il_off), count);
  return launch_status();
}

}  // namespace kfac
