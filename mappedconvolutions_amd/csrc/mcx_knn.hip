// Brute-force k nearest neighbours with a streaming top-k.  The reference
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
#include <initializer_list>

#include "mcx_device.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;

__device__ inline float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ inline double fma_t(double a, double b, double c) { return __builtin_fma(a, b, c); }
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
                                                       int k) {
  const int b = blockIdx.y;
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
    for (int u = 1; u < kBatch; u++) m = ssd[u] < m ? ssd[u] : m;
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
                     dist, (int)D, (int)R, (int)Q, (int)k)
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

}  // namespace
}  // namespace mcx

extern "C" int mcx_knn(const void *ref, const void *query, int64_t *idx, void *dist, int64_t B,
                       int64_t D, int64_t R, int64_t Q, int64_t k, int dtype, void *stream) {
  if (!ref || !query || !idx || !dist) return MCX_E_NULL;
  for (int64_t v : {B, D, R, Q, k, D * R, D * Q})
    if (v <= 0 || v > 0x7fffffffLL) return MCX_E_SHAPE;
  if (k > 64 || B > 65535) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32) return mcx::knn_t<float>(ref, query, idx, dist, B, D, R, Q, k, s);
  if (dtype == MCX_F64) return mcx::knn_t<double>(ref, query, idx, dist, B, D, R, Q, k, s);
  return MCX_E_DTYPE;
}
