// Shape-agnostic scalar kernels for the three products of a mapped convolution
// (gather-product, product-scatter, weight gradient) and the bias gradient.  They
// carry the fp64 instantiation (used by known-answer and gradcheck tests) and any
// fp32 shape the matrix-core kernels do not cover.  Each is written in terms of a
// "plain" operand read at map locations' own index n and a "gathered"/"scattered"
// operand reached through the map, so convolution and transposed convolution share
// them with roles swapped:
//   gather_product : y[b,o,n]  = bias[o] + sum_{g,k} W[o,g,k] * sample(src[b,g], map[n,k])
//       conv forward (o=Co, g=Ci) and transposed-conv backward-input (o=Ci, g=Co)
//   product_scatter: dst[b,d] += splat(sum_s W[s,d,k] * src[b,s,n], map[n,k])
//       conv backward-input (s=Co, d=Ci) and transposed-conv forward (s=Ci, d=Co)
//   weight_grad    : gW[a,g,k] = sum_{b,n} plain[b,a,n] * sample(gath[b,g], map[n,k])
//       conv (a=Co from gy, g=Ci from x) and transposed conv (a=Ci from x, g=Co from gy)
// Reference drivers: src/nn/cuda/mapped_convolution_layer.cu:16-193,
// src/nn/cuda/mapped_transposed_convolution_layer.cu:53-220 and weighted twins.
#include "mcx_conv.h"
#include "mcx_device.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;
constexpr int kOT = 8;  // output channels per thread

template <typename T, int MODE>
__device__ inline T sample_p(const T *plane, const T *map, const T *iw, int64_t e, int P, int h,
                             int w) {
  if (P == 0) {
    Tap<T, MODE> tap;
    tap.set(map[e * 2], map[e * 2 + 1], h, w);
    return tap.gather(plane);
  }
  T acc = T(0);
  for (int p = 0; p < P; p++) {
    Tap<T, MODE> tap;
    tap.set(map[(e + p) * 2], map[(e + p) * 2 + 1], h, w);
    acc += iw[e + p] * tap.gather(plane);
  }
  return acc;
}

template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void gather_product_kernel(
    const T *__restrict__ src, const T *__restrict__ map, const T *__restrict__ iw,
    const T *__restrict__ w, const T *__restrict__ bias, T *__restrict__ y, int G, int O, int SH,
    int SW, int N, int K, int P) {
  const int n = blockIdx.x * kThreads + threadIdx.x;
  if (n >= N) return;
  const int o0 = blockIdx.y * kOT;
  const int b = blockIdx.z;
  const int no = min(kOT, O - o0);
  const int pm = P == 0 ? 1 : P;
  const int64_t plane = (int64_t)SH * SW;
  T acc[kOT];
#pragma unroll
  for (int o = 0; o < kOT; o++) acc[o] = T(0);
  for (int k = 0; k < K; k++) {
    const int64_t e = ((int64_t)n * K + k) * pm;
    for (int g = 0; g < G; g++) {
      const T v = sample_p<T, MODE>(src + ((int64_t)b * G + g) * plane, map, iw, e, P, SH, SW);
#pragma unroll
      for (int o = 0; o < kOT; o++)
        if (o < no) acc[o] += w[((int64_t)(o0 + o) * G + g) * K + k] * v;
    }
  }
#pragma unroll
  for (int o = 0; o < kOT; o++)
    if (o < no) y[((int64_t)b * O + o0 + o) * N + n] = acc[o] + (bias ? bias[o0 + o] : T(0));
}

template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void product_scatter_kernel(
    const T *__restrict__ src, const T *__restrict__ map, const T *__restrict__ iw,
    const T *__restrict__ w, T *__restrict__ dst, int S, int D, int DH, int DW, int N, int K,
    int P) {
  const int n = blockIdx.x * kThreads + threadIdx.x;
  if (n >= N) return;
  const int d0 = blockIdx.y * kOT;
  const int b = blockIdx.z;
  const int nd = min(kOT, D - d0);
  const int pm = P == 0 ? 1 : P;
  const int64_t plane = (int64_t)DH * DW;
  for (int k = 0; k < K; k++) {
    T acc[kOT];
#pragma unroll
    for (int d = 0; d < kOT; d++) acc[d] = T(0);
    for (int s = 0; s < S; s++) {
      const T v = src[((int64_t)b * S + s) * N + n];
#pragma unroll
      for (int d = 0; d < kOT; d++)
        if (d < nd) acc[d] += w[((int64_t)s * D + d0 + d) * K + k] * v;
    }
    const int64_t e = ((int64_t)n * K + k) * pm;
    const int np = P == 0 ? 1 : P;
    for (int p = 0; p < np; p++) {
      Tap<T, MODE> tap;
      tap.set(map[(e + p) * 2], map[(e + p) * 2 + 1], DH, DW);
      const T wp = P == 0 ? T(1) : iw[e + p];
#pragma unroll
      for (int d = 0; d < kOT; d++)
        if (d < nd)
          tap.scatter(dst + ((int64_t)b * D + d0 + d) * plane, P == 0 ? acc[d] : wp * acc[d]);
    }
  }
}

// One workgroup per (g, k) and chunk of kOT plain channels; threads stride over
// (b, n), then reduce through LDS.
template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void weight_grad_kernel(
    const T *__restrict__ plain, const T *__restrict__ gath, const T *__restrict__ map,
    const T *__restrict__ iw, T *__restrict__ gw, int B, int A, int G, int GH, int GW, int N,
    int K, int P) {
  const int g = blockIdx.x / K;
  const int k = blockIdx.x % K;
  const int a0 = blockIdx.y * kOT;
  const int na = min(kOT, A - a0);
  const int pm = P == 0 ? 1 : P;
  const int64_t plane = (int64_t)GH * GW;
  T acc[kOT];
#pragma unroll
  for (int a = 0; a < kOT; a++) acc[a] = T(0);
  for (int b = 0; b < B; b++)
    for (int n = threadIdx.x; n < N; n += kThreads) {
      const int64_t e = ((int64_t)n * K + k) * pm;
      const T v = sample_p<T, MODE>(gath + ((int64_t)b * G + g) * plane, map, iw, e, P, GH, GW);
#pragma unroll
      for (int a = 0; a < kOT; a++)
        if (a < na) acc[a] += plain[((int64_t)b * A + a0 + a) * N + n] * v;
    }
  __shared__ T red[kOT][kThreads];
#pragma unroll
  for (int a = 0; a < kOT; a++) red[a][threadIdx.x] = acc[a];
  __syncthreads();
  for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride)
#pragma unroll
      for (int a = 0; a < kOT; a++) red[a][threadIdx.x] += red[a][threadIdx.x + stride];
    __syncthreads();
  }
  if ((int)threadIdx.x < na) gw[((int64_t)(a0 + threadIdx.x) * G + g) * K + k] = red[threadIdx.x][0];
}

// gb[c] = sum over (b, n) of g[b,c,n]  (grad_output.sum({0,2,3}),
// include/nn/layers/mapped_convolution_layer.h:113).
template <typename T>
__global__ __launch_bounds__(kThreads) void channel_sum_kernel(const T *__restrict__ g,
                                                               T *__restrict__ gb, int B, int C,
                                                               int N) {
  const int c = blockIdx.x;
  T acc = T(0);
  for (int b = 0; b < B; b++) {
    const T *p = g + ((int64_t)b * C + c) * N;
    for (int n = threadIdx.x; n < N; n += kThreads) acc += p[n];
  }
  __shared__ T red[kThreads];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride) red[threadIdx.x] += red[threadIdx.x + stride];
    __syncthreads();
  }
  if (threadIdx.x == 0) gb[c] = red[0];
}

// Two-stage form of the same sum for large tensors: stage 1 reduces one slice of one
// (image, channel) plane per workgroup into part[c][b*splits + s]; stage 2 adds the
// partials of a channel in a fixed order.
template <typename T>
__global__ __launch_bounds__(kThreads) void channel_sum_partial_kernel(
    const T *__restrict__ g, T *__restrict__ part, int C, int N, int splits) {
  const int c = blockIdx.x, b = blockIdx.y, sp = blockIdx.z;
  const int per = (N + splits - 1) / splits;
  const int n0 = sp * per, n1 = min(N, n0 + per);
  const T *p = g + ((int64_t)b * C + c) * N;
  T acc = T(0);
  for (int n = n0 + threadIdx.x; n < n1; n += kThreads) acc += p[n];
  __shared__ T red[kThreads];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride) red[threadIdx.x] += red[threadIdx.x + stride];
    __syncthreads();
  }
  if (threadIdx.x == 0) part[(int64_t)c * gridDim.y * splits + b * splits + sp] = red[0];
}

template <typename T>
__global__ void channel_sum_final_kernel(const T *__restrict__ part, T *__restrict__ gb, int C,
                                         int per_channel) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T acc = T(0);
  for (int i = 0; i < per_channel; i++) acc += part[(int64_t)c * per_channel + i];
  gb[c] = acc;
}

template <typename T>
__global__ void fill_bias_kernel(T *__restrict__ y, const T *__restrict__ bias, int C, int N,
                                 int64_t total) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) y[i] = bias[(i / N) % C];
}

}  // namespace

template <typename T>
int generic_gather_product(const T *src, const T *map, const T *iw, const T *w, const T *bias,
                           T *y, int64_t B, int64_t G, int64_t O, int64_t SH, int64_t SW,
                           int64_t N, int64_t K, int64_t P, int interp, hipStream_t s) {
  dim3 grid(div_up(N, kThreads), div_up(O, kOT), (unsigned)B);
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((gather_product_kernel<T, MODE>), grid,
                                               dim3(kThreads), 0, s, src, map, iw, w, bias, y,
                                               (int)G, (int)O, (int)SH, (int)SW, (int)N, (int)K,
                                               (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T>
int generic_product_scatter(const T *src, const T *map, const T *iw, const T *w, T *dst,
                            int64_t B, int64_t S, int64_t D, int64_t DH, int64_t DW, int64_t N,
                            int64_t K, int64_t P, int interp, hipStream_t s) {
  dim3 grid(div_up(N, kThreads), div_up(D, kOT), (unsigned)B);
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((product_scatter_kernel<T, MODE>), grid,
                                               dim3(kThreads), 0, s, src, map, iw, w, dst, (int)S,
                                               (int)D, (int)DH, (int)DW, (int)N, (int)K, (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T>
int generic_weight_grad(const T *plain, const T *gath, const T *map, const T *iw, T *gw,
                        int64_t B, int64_t A, int64_t G, int64_t GH, int64_t GW, int64_t N,
                        int64_t K, int64_t P, int interp, hipStream_t s) {
  dim3 grid((unsigned)(G * K), div_up(A, kOT));
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((weight_grad_kernel<T, MODE>), grid,
                                               dim3(kThreads), 0, s, plain, gath, map, iw, gw,
                                               (int)B, (int)A, (int)G, (int)GH, (int)GW, (int)N,
                                               (int)K, (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

int channel_sum_splits(int64_t B, int64_t C, int64_t N) {
  if (B * C * N < (1 << 20) || B > 65535) return 0;  // small: one kernel, no scratch
  int splits = 1;
  while (B * C * splits < 2048 && N / (splits * 2) >= 4096 && splits < 64) splits *= 2;
  return splits;
}

size_t channel_sum_scratch_bytes(int64_t B, int64_t C, int64_t N, size_t elem) {
  return (size_t)(B * C * channel_sum_splits(B, C, N)) * elem;
}

template <typename T>
int channel_sum(const T *g, T *gb, T *scratch, int64_t B, int64_t C, int64_t N, hipStream_t s) {
  const int splits = scratch ? channel_sum_splits(B, C, N) : 0;
  if (splits == 0) {
    hipLaunchKernelGGL(channel_sum_kernel<T>, dim3((unsigned)C), dim3(kThreads), 0, s, g, gb,
                       (int)B, (int)C, (int)N);
    MCX_HIP_CHECK_LAUNCH();
    return 0;
  }
  hipLaunchKernelGGL(channel_sum_partial_kernel<T>, dim3((unsigned)C, (unsigned)B, (unsigned)splits),
                     dim3(kThreads), 0, s, g, scratch, (int)C, (int)N, splits);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(channel_sum_final_kernel<T>, dim3((unsigned)((C + 63) / 64)), dim3(64), 0, s,
                     scratch, gb, (int)C, (int)(B * splits));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T>
int fill_bias(T *y, const T *bias, int64_t B, int64_t C, int64_t N, hipStream_t s) {
  const int64_t total = B * C * N;
  const unsigned blocks = (unsigned)std::min<int64_t>((total + 1023) / 1024, 65536);
  hipLaunchKernelGGL(fill_bias_kernel<T>, dim3(blocks), dim3(256), 0, s, y, bias, (int)C, (int)N,
                     total);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

#define MCX_INSTANTIATE(T)                                                                         \
  template int generic_gather_product<T>(const T *, const T *, const T *, const T *, const T *,   \
                                         T *, int64_t, int64_t, int64_t, int64_t, int64_t,        \
                                         int64_t, int64_t, int64_t, int, hipStream_t);            \
  template int generic_product_scatter<T>(const T *, const T *, const T *, const T *, T *,        \
                                          int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,   \
                                          int64_t, int64_t, int, hipStream_t);                    \
  template int generic_weight_grad<T>(const T *, const T *, const T *, const T *, T *, int64_t,   \
                                      int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,       \
                                      int64_t, int, hipStream_t);                                 \
  template int channel_sum<T>(const T *, T *, T *, int64_t, int64_t, int64_t, hipStream_t);       \
  template int fill_bias<T>(T *, const T *, int64_t, int64_t, int64_t, hipStream_t);
MCX_INSTANTIATE(float)
MCX_INSTANTIATE(double)

}  // namespace mcx
