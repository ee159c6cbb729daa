// Bandwidth-bound map-driven gathers and scatters: resample_from_map /
// resample_to_map, mapped max / average pooling and their unpooling adjoints,
// plain and weighted.  One thread owns one map location and a chunk of CH
// channels: the tap (offsets + weights) is resolved once and applied to each of
// the thread's channel planes, so map decoding is amortised and neighbouring lanes
// read neighbouring pixels.
#include "mcx_device.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;
constexpr int kCH = 8;  // channels per thread

enum { OP_RESAMPLE = 0, OP_AVG = 1, OP_MAX = 2 };

// Fill kernel used instead of a memset so that captured graphs replay correctly.
template <typename T>
__global__ void fill_kernel(T *p, int64_t n, T v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

// Gather form.  OP_RESAMPLE: K == 1, out = sample.  OP_AVG: sum of K taps / K.
// OP_MAX: strict-greater running maximum from -FLT_MAX and the winning tap's
// map offset (include/nn/common/mapped_max_pool.h:14-58).
// grid: x over map locations, y over channel chunks, z over images.
template <typename T, int MODE, int OP>
__global__ __launch_bounds__(kThreads) void gather_kernel(
    const T *__restrict__ in, const T *__restrict__ map, const T *__restrict__ iw,
    T *__restrict__ out, int64_t *__restrict__ idx, int C, int IH, int IW, int N, int K, int P) {
  const int n = blockIdx.x * kThreads + threadIdx.x;
  if (n >= N) return;
  const int c0 = blockIdx.y * kCH;
  const int b = blockIdx.z;
  const int64_t plane = (int64_t)IH * IW;
  const T *src = in + ((int64_t)b * C + c0) * plane;
  const int pm = P == 0 ? 1 : P;
  const int nc = min(kCH, C - c0);

  T acc[kCH];
  int64_t best[kCH];
#pragma unroll
  for (int c = 0; c < kCH; c++) {
    acc[c] = OP == OP_MAX ? T(-3.402823466e+38F) : T(0);
    best[c] = -1;
  }
  for (int k = 0; k < K; k++) {
    const int64_t e = ((int64_t)n * K + k) * pm;
    T val[kCH];
    if (P == 0) {
      Tap<T, MODE> tap;
      tap.set(map[e * 2], map[e * 2 + 1], IH, IW);
#pragma unroll
      for (int c = 0; c < kCH; c++)
        if (c < nc) val[c] = tap.gather(src + c * plane);
    } else {
#pragma unroll
      for (int c = 0; c < kCH; c++) val[c] = T(0);
      for (int p = 0; p < P; p++) {
        Tap<T, MODE> tap;
        tap.set(map[(e + p) * 2], map[(e + p) * 2 + 1], IH, IW);
        const T w = iw[e + p];
#pragma unroll
        for (int c = 0; c < kCH; c++)
          if (c < nc) val[c] += w * tap.gather(src + c * plane);
      }
    }
#pragma unroll
    for (int c = 0; c < kCH; c++) {
      if (c >= nc) continue;
      if (OP == OP_MAX) {
        if (val[c] > acc[c]) {
          acc[c] = val[c];
          best[c] = e * 2;
        }
      } else if (OP == OP_AVG) {
        acc[c] += val[c];
      } else {
        acc[c] = val[c];
      }
    }
  }
  const int64_t o = ((int64_t)b * C + c0) * N + n;
#pragma unroll
  for (int c = 0; c < kCH; c++) {
    if (c >= nc) continue;
    out[o + (int64_t)c * N] = OP == OP_AVG ? acc[c] / (T)K : acc[c];
    if (OP == OP_MAX) idx[o + (int64_t)c * N] = best[c];
  }
}

// Scatter form (adjoint of the gather).  OP_RESAMPLE: K == 1, pushes the value;
// OP_AVG: pushes value / K to every tap (include/nn/common/mapped_avg_pool.h:43-70).
template <typename T, int MODE, int OP>
__global__ __launch_bounds__(kThreads) void scatter_kernel(
    const T *__restrict__ in, const T *__restrict__ map, const T *__restrict__ iw,
    T *__restrict__ out, int C, int OH, int OW, int N, int K, int P) {
  const int n = blockIdx.x * kThreads + threadIdx.x;
  if (n >= N) return;
  const int c0 = blockIdx.y * kCH;
  const int b = blockIdx.z;
  const int64_t plane = (int64_t)OH * OW;
  T *dst = out + ((int64_t)b * C + c0) * plane;
  const int pm = P == 0 ? 1 : P;
  const int nc = min(kCH, C - c0);
  const int64_t i0 = ((int64_t)b * C + c0) * N + n;

  T v[kCH];
#pragma unroll
  for (int c = 0; c < kCH; c++) {
    v[c] = c < nc ? in[i0 + (int64_t)c * N] : T(0);
    if (OP == OP_AVG) v[c] = v[c] / (T)K;
  }
  for (int k = 0; k < K; k++) {
    const int64_t e = ((int64_t)n * K + k) * pm;
    if (P == 0) {
      Tap<T, MODE> tap;
      tap.set(map[e * 2], map[e * 2 + 1], OH, OW);
#pragma unroll
      for (int c = 0; c < kCH; c++)
        if (c < nc) tap.scatter(dst + c * plane, v[c]);
    } else {
      for (int p = 0; p < P; p++) {
        Tap<T, MODE> tap;
        tap.set(map[(e + p) * 2], map[(e + p) * 2 + 1], OH, OW);
        const T w = iw[e + p];
#pragma unroll
        for (int c = 0; c < kCH; c++)
          if (c < nc) tap.scatter(dst + c * plane, w * v[c]);
      }
    }
  }
}

// Max unpooling: each pooled pixel sends its gradient through the one tap whose
// map offset was recorded (include/nn/common/mapped_max_pool.h:61-78,135-169).
// The tap differs per channel, so one thread handles one element.
template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void max_unpool_kernel(
    const T *__restrict__ gout, const int64_t *__restrict__ idx, const T *__restrict__ map,
    const T *__restrict__ iw, T *__restrict__ gin, int64_t total, int N, int IH, int IW,
    int64_t map_elems, int P) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t o = idx[i];
  if (o < 0 || o + 1 >= map_elems) return;  // -1: no tap won; also guards corrupt indices
  const int64_t bc = i / N;
  T *dst = gin + bc * (int64_t)IH * IW;
  const T g = gout[i];
  if (P == 0) {
    Tap<T, MODE> tap;
    tap.set(map[o], map[o + 1], IH, IW);
    tap.scatter(dst, g);
  } else {
    for (int p = 0; p < P; p++) {
      Tap<T, MODE> tap;
      tap.set(map[o + 2 * p], map[o + 2 * p + 1], IH, IW);
      tap.scatter(dst, iw[o / 2 + p] * g);
    }
  }
}

bool bad_dims(std::initializer_list<int64_t> dims) {
  for (int64_t d : dims)
    if (d <= 0 || d > 0x7fffffffLL) return true;
  return false;
}

template <typename T>
int fill(T *p, int64_t n, T v, hipStream_t s) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)std::min<int64_t>((n + 1023) / 1024, 65536);
  hipLaunchKernelGGL(fill_kernel<T>, dim3(blocks), dim3(256), 0, s, p, n, v);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T, int OP>
int launch_gather(const void *in, const void *map, const void *iw, void *out, int64_t *idx,
                  int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t N, int64_t K, int64_t P,
                  int interp, hipStream_t s) {
  dim3 grid(div_up(N, kThreads), div_up(C, kCH), (unsigned)B);
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((gather_kernel<T, MODE, OP>), grid, dim3(kThreads),
                                               0, s, (const T *)in, (const T *)map,
                                               (const T *)iw, (T *)out, idx, (int)C, (int)IH,
                                               (int)IW, (int)N, (int)K, (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T, int OP>
int launch_scatter(const void *in, const void *map, const void *iw, void *out, int64_t B,
                   int64_t C, int64_t OH, int64_t OW, int64_t N, int64_t K, int64_t P, int interp,
                   hipStream_t s) {
  int rc = fill<T>((T *)out, B * C * OH * OW, T(0), s);
  if (rc) return rc;
  dim3 grid(div_up(N, kThreads), div_up(C, kCH), (unsigned)B);
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((scatter_kernel<T, MODE, OP>), grid,
                                               dim3(kThreads), 0, s, (const T *)in,
                                               (const T *)map, (const T *)iw, (T *)out, (int)C,
                                               (int)OH, (int)OW, (int)N, (int)K, (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

int check_common(const void *a, const void *map, const void *iw, const void *o, int64_t P,
                 int dtype) {
  if (dtype != MCX_F32 && dtype != MCX_F64) return MCX_E_DTYPE;
  if (!a || !map || !o) return MCX_E_NULL;
  if (P < 0) return MCX_E_SHAPE;
  if ((P == 0) != (iw == nullptr)) return MCX_E_NULL;
  return 0;
}

}  // namespace

// Shared with the convolution translation units.
int fill_f32(float *p, int64_t n, float v, hipStream_t s) { return fill<float>(p, n, v, s); }
int fill_f64(double *p, int64_t n, double v, hipStream_t s) { return fill<double>(p, n, v, s); }

}  // namespace mcx

using namespace mcx;

extern "C" int mcx_resample_from_map(const void *src, const void *map, const void *iw, void *dst,
                                     int64_t B, int64_t C, int64_t SH, int64_t SW, int64_t MH,
                                     int64_t MW, int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(src, map, iw, dst, P, dtype)) return rc;
  if (bad_dims({B, C, SH, SW, MH, MW, SH * SW, MH * MW, MH * MW * (P ? P : 1) * 2}) || B > 65535)
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_RESAMPLE>(src, map, iw, dst, nullptr, B, C, SH, SW, MH * MW, 1,
                                             P, interp, s);
  return launch_gather<double, OP_RESAMPLE>(src, map, iw, dst, nullptr, B, C, SH, SW, MH * MW, 1,
                                            P, interp, s);
}

extern "C" int mcx_resample_to_map(const void *in, const void *map, const void *iw, void *out,
                                   int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                                   int64_t OW, int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, IH * IW, OH * OW, IH * IW * (P ? P : 1) * 2}) || B > 65535)
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_scatter<float, OP_RESAMPLE>(in, map, iw, out, B, C, OH, OW, IH * IW, 1, P,
                                              interp, s);
  return launch_scatter<double, OP_RESAMPLE>(in, map, iw, out, B, C, OH, OW, IH * IW, 1, P, interp,
                                             s);
}

extern "C" int mcx_max_pool(const void *in, const void *map, const void *iw, void *out,
                            int64_t *idx, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                            int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                            void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (!idx) return MCX_E_NULL;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_MAX>(in, map, iw, out, idx, B, C, IH, IW, OH * OW, K, P, interp,
                                        s);
  return launch_gather<double, OP_MAX>(in, map, iw, out, idx, B, C, IH, IW, OH * OW, K, P, interp,
                                       s);
}

extern "C" int mcx_avg_pool(const void *in, const void *map, const void *iw, void *out, int64_t B,
                            int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                            int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_AVG>(in, map, iw, out, nullptr, B, C, IH, IW, OH * OW, K, P,
                                        interp, s);
  return launch_gather<double, OP_AVG>(in, map, iw, out, nullptr, B, C, IH, IW, OH * OW, K, P,
                                       interp, s);
}

extern "C" int mcx_avg_unpool(const void *gout, const void *map, const void *iw, void *gin,
                              int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                              int64_t K, int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(gout, map, iw, gin, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_scatter<float, OP_AVG>(gout, map, iw, gin, B, C, IH, IW, OH * OW, K, P, interp,
                                         s);
  return launch_scatter<double, OP_AVG>(gout, map, iw, gin, B, C, IH, IW, OH * OW, K, P, interp, s);
}

namespace {
template <typename T>
int launch_max_unpool(const void *gout, const int64_t *idx, const void *map, const void *iw,
                      void *gin, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t N,
                      int64_t K, int64_t P, int interp, hipStream_t s) {
  int rc = mcx::fill<T>((T *)gin, B * C * IH * IW, T(0), s);
  if (rc) return rc;
  const int64_t total = B * C * N;
  const int64_t map_elems = N * K * (P ? P : 1) * 2;
  MCX_DISPATCH_MODE(interp,
                    hipLaunchKernelGGL((max_unpool_kernel<T, MODE>), dim3(div_up(total, kThreads)),
                                       dim3(kThreads), 0, s, (const T *)gout, idx, (const T *)map,
                                       (const T *)iw, (T *)gin, total, (int)N, (int)IH, (int)IW,
                                       map_elems, (int)P));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}
}  // namespace

extern "C" int mcx_max_unpool(const void *gout, const int64_t *idx, const void *map,
                              const void *iw, void *gin, int64_t B, int64_t C, int64_t IH,
                              int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                              int dtype, void *stream) {
  if (int rc = check_common(gout, map, iw, gin, P, dtype)) return rc;
  if (!idx) return MCX_E_NULL;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) ||
      B * C * OH * OW > (int64_t)0x7fffffff * kThreads)
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_max_unpool<float>(gout, idx, map, iw, gin, B, C, IH, IW, OH * OW, K, P, interp,
                                    s);
  return launch_max_unpool<double>(gout, idx, map, iw, gin, B, C, IH, IW, OH * OW, K, P, interp, s);
}
