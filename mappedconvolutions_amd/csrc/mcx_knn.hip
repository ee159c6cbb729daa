// k nearest neighbours: a walk over all reference points with a streaming top-k, and (second
// half of the file) a search over a uniform grid for points of one to three dimensions that
// gives the same result bit for bit.  The reference
// (include/util/cuda/knn.cuh:43-275) materialises the R x Q matrix of squared
// distances and insertion-sorts each column with one thread; here one thread owns
// one query, walks the reference points once and keeps its k best in registers,
// so HBM traffic is just the inputs and the [k,Q] outputs.  Reference points are
// read through wave-uniform (scalar) loads: every lane needs the same point.
//
// Contract kept from the reference: squared distance accumulated over the
// dimensions in order with fused multiply-adds, candidates enter only if strictly
// closer than the current k-th and go before the first strictly larger entry (so
// ties keep the lower reference index first), indices are 1-based, distances are
// square-rooted at the end.
#include <algorithm>
#include <cmath>
#include <initializer_list>

#include "mcx_device.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;

__host__ __device__ constexpr size_t align_up256(size_t v) { return (v + 255) & ~(size_t)255; }

// Grid search (second half of this file): per batch element, at the start of its workspace slice
template <typename T>
struct GridHead {
  T lo[3], inv_h[3], h[3];
  int skewed;  // nonzero: a quarter of the points share one cell; the plain walk runs instead
};
template <typename T>
struct alignas(sizeof(T) * 4) GridPoint {
  T c[3];
  int idx;  // 1-based index of the reference point
};

__device__ inline float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ inline double fma_t(double a, double b, double c) { return __builtin_fma(a, b, c); }
__device__ inline float min_t(float a, float b) { return __builtin_fminf(a, b); }
__device__ inline double min_t(double a, double b) { return __builtin_fmin(a, b); }
__device__ inline float sqrt_t(float v) { return sqrtf(v); }
__device__ inline double sqrt_t(double v) { return sqrt(v); }

template <typename T>
__device__ inline T inf_t() { return (T)__builtin_huge_valf(); }

// DT > 0: compile-time dimension, query coordinates live in registers.
// DT == 0: any dimension, coordinates re-read from memory (slow path).
template <typename T, int KMAX, int DT>
__global__ __launch_bounds__(kThreads) void knn_kernel(const T *__restrict__ ref,
                                                       const T *__restrict__ query,
                                                       int64_t *__restrict__ idx,
                                                       T *__restrict__ dist, int D, int R, int Q,
                                                       int k, const char *__restrict__ grid_ws,
                                                       size_t grid_slice) {
  const int b = blockIdx.y;
  // launched behind a grid search: only for batch elements whose grid was not worth walking
  if (grid_ws &&
      !reinterpret_cast<const GridHead<T> *>(grid_ws + (size_t)b * grid_slice)->skewed)
    return;
  const int q = blockIdx.x * kThreads + threadIdx.x;
  const bool live = q < Q;
  const int qc = live ? q : Q - 1;
  const T *rb = ref + (int64_t)b * D * R;
  const T *qb = query + (int64_t)b * D * Q;

  T qv[DT > 0 ? DT : 1];
#pragma unroll
  for (int d = 0; d < DT; d++) qv[d] = qb[(int64_t)d * Q + qc];

  T bd[KMAX];
  int bi[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; j++) {
    bd[j] = inf_t<T>();
    bi[j] = 0;
  }

  auto ssd_of = [&](int r) {
    T ssd = T(0);
    if (DT > 0) {
#pragma unroll
      for (int d = 0; d < DT; d++) {
        const T t = rb[(int64_t)d * R + r] - qv[d];
        ssd = fma_t(t, t, ssd);
      }
    } else {
      for (int d = 0; d < D; d++) {
        const T t = rb[(int64_t)d * R + r] - qb[(int64_t)d * Q + qc];
        ssd = fma_t(t, t, ssd);
      }
    }
    return ssd;
  };
  auto insert = [&](T ssd, int r) {
    if (ssd < bd[KMAX - 1]) {
      T cd = ssd;
      int ci = r + 1;
      bool shifting = false;
#pragma unroll
      for (int j = 0; j < KMAX; j++) {
        shifting = shifting || (cd < bd[j]);
        if (shifting) {
          const T td = bd[j];
          const int ti = bi[j];
          bd[j] = cd;
          bi[j] = ci;
          cd = td;
          ci = ti;
        }
      }
    }
  };
  // Reference points are taken kBatch at a time: their distances are independent work
  // (the wave-uniform loads of the next points overlap the arithmetic), and a single
  // comparison of the batch minimum decides whether any lane has to insert at all.
  constexpr int kBatch = 8;
  int r = 0;
  for (; r + kBatch <= R; r += kBatch) {
    T ssd[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; u++) ssd[u] = ssd_of(r + u);
    T m = ssd[0];
#pragma unroll
    for (int u = 1; u < kBatch; u++) m = min_t(m, ssd[u]);  // (a NaN yields to a number)
    if (m < bd[KMAX - 1]) {
#pragma unroll
      for (int u = 0; u < kBatch; u++) insert(ssd[u], r + u);  // in index order: ties keep it
    }
  }
  for (; r < R; r++) insert(ssd_of(r), r);
  if (!live) return;
#pragma unroll
  for (int j = 0; j < KMAX; j++) {
    if (j < k) {
      const int64_t o = ((int64_t)b * k + j) * Q + q;
      idx[o] = bi[j];
      dist[o] = bi[j] > 0 ? sqrt_t(bd[j]) : T(0);
    }
  }
}

template <typename T, int KMAX>
int launch_knn(const T *ref, const T *query, int64_t *idx, T *dist, int64_t B, int64_t D,
               int64_t R, int64_t Q, int64_t k, hipStream_t s) {
  dim3 grid(div_up(Q, kThreads), (unsigned)B);
#define MCX_KNN_LAUNCH(DT)                                                                        \
  hipLaunchKernelGGL((knn_kernel<T, KMAX, DT>), grid, dim3(kThreads), 0, s, ref, query, idx,     \
                     dist, (int)D, (int)R, (int)Q, (int)k, (const char *)nullptr, (size_t)0)
  switch (D) {
    case 1: MCX_KNN_LAUNCH(1); break;
    case 2: MCX_KNN_LAUNCH(2); break;
    case 3: MCX_KNN_LAUNCH(3); break;
    case 4: MCX_KNN_LAUNCH(4); break;
    default: MCX_KNN_LAUNCH(0); break;
  }
#undef MCX_KNN_LAUNCH
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T>
int knn_t(const void *ref, const void *query, int64_t *idx, void *dist, int64_t B, int64_t D,
          int64_t R, int64_t Q, int64_t k, hipStream_t s) {
  const T *r = (const T *)ref, *q = (const T *)query;
  T *d = (T *)dist;
  if (k <= 8) return launch_knn<T, 8>(r, q, idx, d, B, D, R, Q, k, s);
  if (k <= 16) return launch_knn<T, 16>(r, q, idx, d, B, D, R, Q, k, s);
  if (k <= 32) return launch_knn<T, 32>(r, q, idx, d, B, D, R, Q, k, s);
  return launch_knn<T, 64>(r, q, idx, d, B, D, R, Q, k, s);
}


// ---------------------------------------------------------------------------------
// Grid search for points of one to three dimensions: the same result, bit for bit, as the
// walk over all reference points above (same distance arithmetic, same order (distance,
// index) of the k kept), found among the reference points of the grid cells around the
// query only.  The reference points are binned into a uniform grid over their bounding box
// (count, prefix sum, fill); a query walks the cells around its own in rings of growing
// Chebyshev radius and stops once its k-th distance is safely below the distance to the
// nearest face of the cube of cells it has seen (every point not seen lies beyond a face).
// Points arrive in no particular order, so ties are resolved by the index explicitly.
// Reference points with a non-finite coordinate can never enter a result (their distance
// is not smaller than anything) and are left out of the grid.
// ---------------------------------------------------------------------------------
constexpr int kGridThreads = 1024;

#ifndef MCX_KNN_CELLS_PER_POINT
#define MCX_KNN_CELLS_PER_POINT 2.0
#endif
constexpr double kCellsPerPoint = MCX_KNN_CELLS_PER_POINT;
struct GridShape {
  int g[3];
  int64_t cells;
};
// Cells per dimension from the number of points alone (about two points per cell of a
// uniformly filled box; the host needs the workspace size before any data is seen).
inline GridShape grid_shape(int64_t D, int64_t R) {
  GridShape s{{1, 1, 1}, 1};
  const double per = std::pow((double)std::max<int64_t>(R, 1) * kCellsPerPoint, 1.0 / (double)D);
  const int cap = D == 1 ? 65536 : D == 2 ? 512 : 64;
  const int g = (int)std::min<double>(cap, std::max(1.0, std::ceil(per)));
  for (int d = 0; d < (int)D; d++) s.g[d] = g;
  s.cells = (int64_t)s.g[0] * s.g[1] * s.g[2];
  return s;
}
template <typename T>
size_t grid_slice_bytes(int64_t D, int64_t R) {
  const GridShape s = grid_shape(D, R);
  return align_up256(sizeof(GridHead<T>)) + align_up256((size_t)(s.cells + 1) * 4) +
         align_up256((size_t)s.cells * 4) + align_up256((size_t)R * sizeof(GridPoint<T>));
}

template <typename T>
__device__ inline bool finite_t(T v) { return v - v == T(0); }

template <typename T, int D>
__device__ inline int cell_of(const GridHead<T> &h, const int *g, const T *c, int *cd) {
  int cell = 0;
#pragma unroll
  for (int d = D - 1; d >= 0; d--) {
    const int i = min(max((int)floor((c[d] - h.lo[d]) * h.inv_h[d]), 0), g[d] - 1);
    cd[d] = i;
    cell = cell * g[d] + i;
  }
  return cell;
}

// One workgroup per batch element: bounding box of the finite reference points, cell size,
// counters cleared.
template <typename T, int D>
__global__ __launch_bounds__(kGridThreads) void knn_grid_box_kernel(
    const T *__restrict__ ref, char *__restrict__ ws, size_t slice, int R, int g0, int g1, int g2,
    int cells) {
  __shared__ T smin[D][kGridThreads / 64], smax[D][kGridThreads / 64];
  const int b = blockIdx.x;
  const T *rb = ref + (int64_t)b * D * R;
  char *base = ws + (size_t)b * slice;
  GridHead<T> *head = reinterpret_cast<GridHead<T> *>(base);
  int *start = reinterpret_cast<int *>(base + align_up256(sizeof(GridHead<T>)));
  int *cursor = reinterpret_cast<int *>(reinterpret_cast<char *>(start) +
                                        align_up256((size_t)(cells + 1) * 4));
  T mn[D], mx[D];
#pragma unroll
  for (int d = 0; d < D; d++) {
    mn[d] = inf_t<T>();
    mx[d] = -inf_t<T>();
  }
  for (int r = threadIdx.x; r < R; r += kGridThreads) {
    T c[D];
    bool ok = true;
#pragma unroll
    for (int d = 0; d < D; d++) {
      c[d] = rb[(int64_t)d * R + r];
      ok = ok && finite_t(c[d]);
    }
    if (ok) {
#pragma unroll
      for (int d = 0; d < D; d++) {
        mn[d] = c[d] < mn[d] ? c[d] : mn[d];
        mx[d] = c[d] > mx[d] ? c[d] : mx[d];
      }
    }
  }
#pragma unroll
  for (int d = 0; d < D; d++) {
    for (int o = 32; o > 0; o >>= 1) {
      const T a = __shfl_xor(mn[d], o), c = __shfl_xor(mx[d], o);
      mn[d] = a < mn[d] ? a : mn[d];
      mx[d] = c > mx[d] ? c : mx[d];
    }
    if ((threadIdx.x & 63) == 0) {
      smin[d][threadIdx.x >> 6] = mn[d];
      smax[d][threadIdx.x >> 6] = mx[d];
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int g[3] = {g0, g1, g2};
    for (int d = 0; d < 3; d++) {
      T lo = T(0), hi = T(0);
      if (d < D) {
        lo = smin[d][0];
        hi = smax[d][0];
        for (int w = 1; w < kGridThreads / 64; w++) {
          lo = smin[d][w] < lo ? smin[d][w] : lo;
          hi = smax[d][w] > hi ? smax[d][w] : hi;
        }
      }
      const T width = hi - lo;  // not finite: no finite point, or the box overflows
      const bool usable = d < D && width > T(0) && finite_t(width);
      head->lo[d] = usable ? lo : T(0);
      head->h[d] = usable ? width / (T)g[d] : T(0);
      head->inv_h[d] = usable ? (T)g[d] / width : T(0);  // unusable: everything in cell 0
    }
    head->skewed = 0;
  }
  for (int c = threadIdx.x; c < cells; c += kGridThreads) {
    start[c] = 0;
    cursor[c] = 0;
  }
  if (threadIdx.x == 0) start[cells] = 0;
}

template <typename T, int D>
__global__ __launch_bounds__(256) void knn_grid_count_kernel(const T *__restrict__ ref,
                                                            char *__restrict__ ws, size_t slice,
                                                            int R, int g0, int g1, int g2,
                                                            int cells, int fill) {
  const int b = blockIdx.y;
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r >= R) return;
  const T *rb = ref + (int64_t)b * D * R;
  char *base = ws + (size_t)b * slice;
  const GridHead<T> &head = *reinterpret_cast<const GridHead<T> *>(base);
  int *start = reinterpret_cast<int *>(base + align_up256(sizeof(GridHead<T>)));
  int *cursor = reinterpret_cast<int *>(reinterpret_cast<char *>(start) +
                                        align_up256((size_t)(cells + 1) * 4));
  GridPoint<T> *pts = reinterpret_cast<GridPoint<T> *>(reinterpret_cast<char *>(cursor) +
                                                       align_up256((size_t)cells * 4));
  const int g[3] = {g0, g1, g2};
  T c[3] = {T(0), T(0), T(0)};
  bool ok = true;
#pragma unroll
  for (int d = 0; d < D; d++) {
    c[d] = rb[(int64_t)d * R + r];
    ok = ok && finite_t(c[d]);
  }
  if (!ok) return;
  int cd[3];
  const int cell = cell_of<T, D>(head, g, c, cd);
  if (!fill) {
    atomicAdd(&start[cell], 1);  // counts now, offsets after the scan
  } else {
    GridPoint<T> p;
    p.c[0] = c[0]; p.c[1] = c[1]; p.c[2] = c[2];
    p.idx = r + 1;
    pts[start[cell] + atomicAdd(&cursor[cell], 1)] = p;
  }
}

// counts -> offsets (exclusive prefix sum, start[cells] = number of binned points), one
// workgroup per batch element, 1024 cells per step; also decides whether the grid is worth
// walking.
template <typename T>
__global__ __launch_bounds__(kGridThreads) void knn_grid_scan_kernel(char *__restrict__ ws,
                                                                    size_t slice, int cells,
                                                                    int R) {
  __shared__ int wave_sum[kGridThreads / 64];
  __shared__ int biggest[kGridThreads / 64];
  char *base = ws + (size_t)blockIdx.x * slice;
  GridHead<T> *head = reinterpret_cast<GridHead<T> *>(base);
  int *start = reinterpret_cast<int *>(base + align_up256(sizeof(GridHead<T>)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int carry = 0, big = 0;
  // four consecutive cells per thread and step (the slice is 256-byte aligned and padded, so
  // 16-byte accesses past `cells` stay inside it); the next step's counts are fetched before
  // this step's barriers
  constexpr int kStep = kGridThreads * 4;
  int4 *cell4 = reinterpret_cast<int4 *>(start);
  auto fetch = [&](int c0) {
    const int c = c0 + threadIdx.x * 4;
    int4 v = c < cells ? cell4[c >> 2] : make_int4(0, 0, 0, 0);
    if (c + 1 >= cells) v.y = 0;
    if (c + 2 >= cells) v.z = 0;
    if (c + 3 >= cells) v.w = 0;
    return v;
  };
  int4 next = fetch(0);
  for (int c0 = 0; c0 < cells; c0 += kStep) {
    const int c = c0 + threadIdx.x * 4;
    const int4 v = next;
    if (c0 + kStep < cells) next = fetch(c0 + kStep);
    big = max(max(big, max(v.x, v.y)), max(v.z, v.w));
    const int mine = v.x + v.y + v.z + v.w;
    int incl = mine;  // inclusive scan within the wave
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(incl, o);
      if (lane >= o) incl += t;
    }
    __syncthreads();  // the previous step's wave sums have been read
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry, total = 0;
    for (int w = 0; w < kGridThreads / 64; w++) {
      const int t = wave_sum[w];
      if (w < wave) before += t;
      total += t;
    }
    if (c < cells) {  // (entries past `cells` inside the last 16 bytes are padding or start[cells])
      int4 o;
      o.x = before + incl - mine;
      o.y = o.x + v.x;
      o.z = o.y + v.y;
      o.w = o.z + v.z;
      if (c + 3 < cells) {
        cell4[c >> 2] = o;
      } else {
        start[c] = o.x;
        if (c + 1 < cells) start[c + 1] = o.y;
        if (c + 2 < cells) start[c + 2] = o.z;
      }
    }
    carry += total;
  }
  for (int o = 32; o > 0; o >>= 1) big = max(big, __shfl_xor(big, o));
  __syncthreads();
  if (lane == 0) biggest[wave] = big;
  __syncthreads();
  if (threadIdx.x == 0) {
    start[cells] = carry;
    int m = 0;
    for (int w = 0; w < kGridThreads / 64; w++) m = max(m, biggest[w]);
    head->skewed = m > max(256, R / 4) ? 1 : 0;
  }
}

template <typename T, int KMAX, int D>
__global__ __launch_bounds__(kThreads) void knn_grid_kernel(
    const T *__restrict__ query, int64_t *__restrict__ idx, T *__restrict__ dist,
    const char *__restrict__ ws, size_t slice, int Q, int k, int g0, int g1, int g2, int cells) {
  const int b = blockIdx.y;
  const char *base = ws + (size_t)b * slice;
  const GridHead<T> head = *reinterpret_cast<const GridHead<T> *>(base);
  if (head.skewed) return;
  const int *start = reinterpret_cast<const int *>(base + align_up256(sizeof(GridHead<T>)));
  const GridPoint<T> *pts = reinterpret_cast<const GridPoint<T> *>(
      reinterpret_cast<const char *>(start) + align_up256((size_t)(cells + 1) * 4) +
      align_up256((size_t)cells * 4));
  const int q = blockIdx.x * kThreads + threadIdx.x;
  if (q >= Q) return;
  const T *qb = query + (int64_t)b * D * Q;
  const int g[3] = {g0, g1, g2};

  T qv[3] = {T(0), T(0), T(0)};
  bool finite = true;
#pragma unroll
  for (int d = 0; d < D; d++) {
    qv[d] = qb[(int64_t)d * Q + q];
    finite = finite && finite_t(qv[d]);
  }
  T bd[KMAX];
  int bi[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; j++) {
    bd[j] = inf_t<T>();
    bi[j] = 0;
  }
  // (cd, ci) goes before (d, i): closer, or as close with the lower index; an empty slot
  // (infinite distance, index 0) yields to any finite distance only
  auto before = [](T cd, int ci, T d, int i) { return cd < d || (cd == d && ci < i); };
  auto insert = [&](T ssd, int pi) {
    if (before(ssd, pi, bd[KMAX - 1], bi[KMAX - 1])) {
      T cd = ssd;
      int ci = pi;
      bool shifting = false;
#pragma unroll
      for (int j = 0; j < KMAX; j++) {
        shifting = shifting || before(cd, ci, bd[j], bi[j]);
        if (shifting) {
          const T td = bd[j];
          const int ti = bi[j];
          bd[j] = cd;
          bi[j] = ci;
          cd = td;
          ci = ti;
        }
      }
    }
  };
  // The points of cells cell_a .. cell_b, four at a time so that their loads are in flight
  // together (a load past the run re-reads its last point and is not used).
  constexpr int kUnroll = 4;
  auto scan = [&](int cell_a, int cell_b) {
    const int e = start[cell_b + 1];
    for (int r = start[cell_a]; r < e; r += kUnroll) {
      GridPoint<T> p[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) p[u] = pts[min(r + u, e - 1)];
      T ssd[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) {
        ssd[u] = T(0);
#pragma unroll
        for (int d = 0; d < D; d++) {
          const T t = p[u].c[d] - qv[d];
          ssd[u] = fma_t(t, t, ssd[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; u++)
        if (r + u < e) insert(ssd[u], p[u].idx);
    }
  };

  if (finite && start[cells] > 0) {  // a query with a non-finite coordinate is near nothing
    int c[3] = {0, 0, 0};
    cell_of<T, D>(head, g, qv, c);
    // a dimension the points do not spread over (cell size 0) has them all in its cell 0
    int ge[3] = {1, 1, 1};
    T hmin = inf_t<T>();
    // largest coordinate magnitude of a cell face: the face lo + n * h is rounded to one unit in
    // the last place of that magnitude, and the cell index floor((c - lo) / h) of a point next to
    // face n is off by a few units in the last place of n, i.e. of (n * h) in coordinates
    T reach = T(0);
#pragma unroll
    for (int d = 0; d < D; d++) {
      if (head.h[d] > T(0)) {
        ge[d] = g[d];
        hmin = head.h[d] < hmin ? head.h[d] : hmin;
        const T lo = head.lo[d] < T(0) ? -head.lo[d] : head.lo[d];
        const T span = (T)g[d] * head.h[d];
        reach = lo + span > reach ? lo + span : reach;
      }
    }
    const int gmax = max(ge[0], max(ge[1], ge[2]));
    constexpr T kUlp = sizeof(T) == 4 ? T(1.1920929e-7) : T(2.220446049250313e-16);
    // a thousandth of a cell, plus the rounding above (which outgrows it on long one-dimensional
    // grids: 65536 cells in fp32 put a face off by hundredths of a cell)
    const T slack = hmin * T(1e-3) + T(16) * kUlp * reach;
    for (int rho = 0; rho < gmax; rho++) {
      // ring rho: rows of cells along the first dimension; rows on the ring's outer faces
      // are contiguous runs of cells (one run of points), the others contribute their ends
      const int z0 = max(c[2] - rho, 0), z1 = min(c[2] + rho, ge[2] - 1);
      const int y0 = max(c[1] - rho, 0), y1 = min(c[1] + rho, ge[1] - 1);
      const int xa = c[0] - rho, xb = c[0] + rho;
      for (int z = z0; z <= z1; z++) {
        for (int y = y0; y <= y1; y++) {
          const int row = (z * g1 + y) * g0;
          const bool face = (D > 2 && (z == c[2] - rho || z == c[2] + rho)) ||
                            (D > 1 && (y == c[1] - rho || y == c[1] + rho));
          if (face || rho == 0) {
            scan(row + max(xa, 0), row + min(xb, ge[0] - 1));
          } else {
            if (xa >= 0) scan(row + xa, row + xa);
            if (xb < ge[0]) scan(row + xb, row + xb);
          }
        }
      }
      // every point not seen lies beyond a face of the cube of cells seen that is not on the
      // grid's boundary; m: distance from the query to the nearest such face
      T m = inf_t<T>();
#pragma unroll
      for (int d = 0; d < D; d++) {
        if (c[d] - rho > 0) {
          const T f = head.lo[d] + (T)(c[d] - rho) * head.h[d];
          m = qv[d] - f < m ? qv[d] - f : m;
        }
        if (c[d] + rho < ge[d] - 1) {
          const T f = head.lo[d] + (T)(c[d] + rho + 1) * head.h[d];
          m = f - qv[d] < m ? f - qv[d] : m;
        }
      }
      if (!(m < inf_t<T>())) break;  // the whole grid has been seen
      T kth = bd[0];
#pragma unroll
      for (int j = 1; j < KMAX; j++) kth = j < k ? bd[j] : kth;
      // (the margins cover the rounding of cell assignment, faces and distances)
      const T safe = m - slack;
      if (safe > T(0) && kth < safe * safe * T(1.0 - 1e-5)) break;
    }
  }
#pragma unroll
  for (int j = 0; j < KMAX; j++) {
    if (j < k) {
      const int64_t o = ((int64_t)b * k + j) * Q + q;
      idx[o] = bi[j];
      dist[o] = bi[j] > 0 ? sqrt_t(bd[j]) : T(0);
    }
  }
}

template <typename T, int KMAX, int D>
int launch_knn_grid(const T *ref, const T *query, int64_t *idx, T *dist, void *workspace,
                    int64_t B, int64_t R, int64_t Q, int64_t k, hipStream_t s) {
  const GridShape gs = grid_shape(D, R);
  const size_t slice = grid_slice_bytes<T>(D, R);
  char *ws = (char *)workspace;
  const int cells = (int)gs.cells;
  hipLaunchKernelGGL((knn_grid_box_kernel<T, D>), dim3((unsigned)B), dim3(kGridThreads), 0, s, ref,
                     ws, slice, (int)R, gs.g[0], gs.g[1], gs.g[2], cells);
  MCX_HIP_CHECK_LAUNCH();
  const dim3 rgrid(div_up(R, 256), (unsigned)B);
  hipLaunchKernelGGL((knn_grid_count_kernel<T, D>), rgrid, dim3(256), 0, s, ref, ws, slice, (int)R,
                     gs.g[0], gs.g[1], gs.g[2], cells, 0);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(knn_grid_scan_kernel<T>, dim3((unsigned)B), dim3(kGridThreads), 0, s, ws,
                     slice, cells, (int)R);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL((knn_grid_count_kernel<T, D>), rgrid, dim3(256), 0, s, ref, ws, slice, (int)R,
                     gs.g[0], gs.g[1], gs.g[2], cells, 1);
  MCX_HIP_CHECK_LAUNCH();
  const dim3 qgrid(div_up(Q, kThreads), (unsigned)B);
  hipLaunchKernelGGL((knn_grid_kernel<T, KMAX, D>), qgrid, dim3(kThreads), 0, s, query, idx, dist,
                     ws, slice, (int)Q, (int)k, gs.g[0], gs.g[1], gs.g[2], cells);
  MCX_HIP_CHECK_LAUNCH();
  // the plain walk, for batch elements whose grid came out skewed (it returns at once otherwise)
  hipLaunchKernelGGL((knn_kernel<T, KMAX, D>), qgrid, dim3(kThreads), 0, s, ref, query, idx, dist,
                     (int)D, (int)R, (int)Q, (int)k, (const char *)ws, slice);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

// The grid pays once there are enough reference points to skip.
inline bool grid_applies(int64_t D, int64_t R) { return D >= 1 && D <= 3 && R >= 512; }

template <typename T>
int knn_grid_t(const void *ref, const void *query, int64_t *idx, void *dist, void *workspace,
               int64_t B, int64_t D, int64_t R, int64_t Q, int64_t k, hipStream_t s) {
  const T *r = (const T *)ref, *q = (const T *)query;
  T *d = (T *)dist;
#define MCX_KNN_GRID(KMAX)                                                                  \
  switch (D) {                                                                              \
    case 1: return launch_knn_grid<T, KMAX, 1>(r, q, idx, d, workspace, B, R, Q, k, s);     \
    case 2: return launch_knn_grid<T, KMAX, 2>(r, q, idx, d, workspace, B, R, Q, k, s);     \
    default: return launch_knn_grid<T, KMAX, 3>(r, q, idx, d, workspace, B, R, Q, k, s);    \
  }
  if (k <= 8) { MCX_KNN_GRID(8) }
  if (k <= 16) { MCX_KNN_GRID(16) }
  if (k <= 32) { MCX_KNN_GRID(32) }
  MCX_KNN_GRID(64)
#undef MCX_KNN_GRID
}

}  // namespace
}  // namespace mcx

extern "C" size_t mcx_knn_workspace(int64_t B, int64_t D, int64_t R, int dtype) {
  if (B <= 0 || R <= 0 || !mcx::grid_applies(D, R)) return 0;
  if (dtype == MCX_F32) return (size_t)B * mcx::grid_slice_bytes<float>(D, R);
  if (dtype == MCX_F64) return (size_t)B * mcx::grid_slice_bytes<double>(D, R);
  return 0;
}

extern "C" int mcx_knn(const void *ref, const void *query, int64_t *idx, void *dist,
                       void *workspace, size_t workspace_bytes, int64_t B, int64_t D, int64_t R,
                       int64_t Q, int64_t k, int dtype, void *stream) {
  if (!ref || !query || !idx || !dist) return MCX_E_NULL;
  for (int64_t v : {B, D, R, Q, k, D * R, D * Q})
    if (v <= 0 || v > 0x7fffffffLL) return MCX_E_SHAPE;
  if (k > 64 || B > 65535) return MCX_E_SHAPE;
  if (dtype != MCX_F32 && dtype != MCX_F64) return MCX_E_DTYPE;
  hipStream_t s = (hipStream_t)stream;
  const size_t need = mcx_knn_workspace(B, D, R, dtype);
  if (workspace && need > 0) {
    if (workspace_bytes < need) return MCX_E_WORKSPACE;
    if (dtype == MCX_F32)
      return mcx::knn_grid_t<float>(ref, query, idx, dist, workspace, B, D, R, Q, k, s);
    return mcx::knn_grid_t<double>(ref, query, idx, dist, workspace, B, D, R, Q, k, s);
  }
  if (dtype == MCX_F32) return mcx::knn_t<float>(ref, query, idx, dist, B, D, R, Q, k, s);
  return mcx::knn_t<double>(ref, query, idx, dist, B, D, R, Q, k, s);
}
