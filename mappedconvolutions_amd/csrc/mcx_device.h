// Device-side building blocks shared by every kernel of the mapped-convolution
// backend: the three interpolators (gather and scatter form), atomics and launch
// helpers.  Semantics follow the reference's include/core/interpolation.h:85-238
// and include/core/resample.h:34-162; the formulation (precomputed "taps" that
// are reused across channels) is specific to this backend.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mcx.h"

namespace mcx {

constexpr int kInterpNearest = 0;
constexpr int kInterpBilinear = 1;
constexpr int kInterpBispherical = 2;

// Any interpolation code other than 1 or 2 means nearest (include/core/resample.h:69-71).
__host__ __device__ inline int canonical_interp(int interp) {
  return (interp == kInterpBilinear || interp == kInterpBispherical) ? interp : kInterpNearest;
}

#define MCX_HIP_CHECK_LAUNCH()                      \
  do {                                              \
    hipError_t e__ = hipGetLastError();             \
    if (e__ != hipSuccess) return (int)e__;         \
  } while (0)

// ---- scalar helpers -------------------------------------------------------

__device__ inline float mcx_floor(float v) { return floorf(v); }
__device__ inline double mcx_floor(double v) { return floor(v); }
__device__ inline float mcx_trunc(float v) { return truncf(v); }
__device__ inline double mcx_trunc(double v) { return trunc(v); }
__device__ inline float mcx_abs(float v) { return fabsf(v); }
__device__ inline double mcx_abs(double v) { return fabs(v); }

// llround(double(v)) of include/core/interpolation.h:90-91: halves go away from
// zero.  v - trunc(v) is exact, so no double rounding can occur (adding 0.5 and
// truncating would round 0.49999997f up).
template <typename T>
__device__ inline T round_half_away(T v) {
  T t = mcx_trunc(v);
  const T frac = v - t;
  if (mcx_abs(frac) >= T(0.5)) t += (v < T(0)) ? T(-1) : T(1);
  return t;
}

// Saturating conversion of an already integral floating value.
__device__ inline int to_int(float v) { return (int)fminf(fmaxf(v, -2.0e9f), 2.0e9f); }
__device__ inline int to_int(double v) { return (int)fmin(fmax(v, -2.0e9), 2.0e9); }

__device__ inline float mcx_fma(float a, float b, float c) { return fmaf(a, b, c); }
__device__ inline double mcx_fma(double a, double b, double c) { return fma(a, b, c); }

__device__ inline int wrap_index(int v, int n) {
  int r = v % n;
  return r < 0 ? r + n : r;
}

__device__ inline void atomic_add(float *p, float v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void atomic_add(double *p, double v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Element `off` of a plane, or element 0 when off < 0 (the caller discards that value).  The
// load itself is unconditional: a load behind a per-lane test becomes a branch, and a chain of
// such branches keeps a thread's loads from being in flight together.  The address is the
// plane pointer (wave-uniform where the plane is chosen per workgroup) plus a 32-bit byte
// offset, so planes are limited to 4 GiB.
template <typename TD>
__device__ inline TD load_elem(const TD *plane, int off) {
  const unsigned byte_off = (off < 0 ? 0u : (unsigned)off) * (unsigned)sizeof(TD);
  return *reinterpret_cast<const TD *>(reinterpret_cast<const char *>(plane) + byte_off);
}

// A plane as a buffer resource: base pointer and size in bytes.  A load whose byte offset
// lies beyond the size returns 0 and touches no memory, so a tap's corners outside the plane
// (or with weight zero) are given the offset kOobOffset: no test, no select, no traffic.  The
// descriptor lives in scalar registers; planes are limited to kOobOffset bytes.
typedef __amdgpu_buffer_rsrc_t plane_buf_t;
constexpr unsigned kOobOffset = 0xffffff00u;
__device__ inline plane_buf_t plane_buf(const void *plane, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(plane), (short)0, (int)bytes,
                                           0x00020000);
}
__device__ inline float buf_load(plane_buf_t r, unsigned byte_off, float) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}
__device__ inline double buf_load(plane_buf_t r, unsigned byte_off, double) {
  return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, 0));
}
// Stores through a buffer resource: one whose byte offset lies beyond the size is dropped, so
// a lane with nothing to store passes kOobOffset instead of branching around the store.
typedef unsigned buf_u32x2 __attribute__((ext_vector_type(2)));
__device__ inline void buf_store(plane_buf_t r, unsigned byte_off, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, (int)byte_off, 0, 0);
}
__device__ inline void buf_store(plane_buf_t r, unsigned byte_off, double v) {
  __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(buf_u32x2, v), r, (int)byte_off, 0, 0);
}
__device__ inline void buf_store(plane_buf_t r, unsigned byte_off, int64_t v) {
  __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(buf_u32x2, v), r, (int)byte_off, 0, 0);
}
// Two neighbouring elements with one load (the address need only be element-aligned).
struct float_pair { float x, y; };
struct double_pair { double x, y; };
__device__ inline float_pair buf_load_pair(plane_buf_t r, unsigned byte_off, float) {
  return __builtin_bit_cast(float_pair, __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, 0));
}
__device__ inline double_pair buf_load_pair(plane_buf_t r, unsigned byte_off, double) {
  return __builtin_bit_cast(double_pair,
                            __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
}

// ---- taps -----------------------------------------------------------------
// A tap is one (x, y) sample location resolved against an H x W plane: up to
// four in-plane element offsets and their weights.  Offsets are -1 for corners
// that fall outside the plane (they contribute exactly zero).  Because the map is
// shared by every channel and image, a tap is computed once and applied to many
// planes.
template <typename T, int MODE>
struct Tap;

template <typename T>
struct Tap<T, kInterpNearest> {
  int off;
  __device__ inline void set(T x, T y, int h, int w) {
    const int xi = to_int(round_half_away(x));
    const int yi = to_int(round_half_away(y));
    const bool ok = xi >= 0 && xi <= w - 1 && yi >= 0 && yi <= h - 1;
    off = ok ? yi * w + xi : -1;
  }
  template <typename TD>
  __device__ inline T gather(const TD *plane) const {
    const T d = (T)load_elem(plane, off);
    return off >= 0 ? d : T(0);
  }
  __device__ inline T gather(plane_buf_t plane) const {
    return buf_load(plane, off < 0 ? kOobOffset : (unsigned)off * (unsigned)sizeof(T), T());
  }
  // gather() in two steps, so that a caller can issue the loads of many taps before it
  // uses any of them
  __device__ inline void load(plane_buf_t plane, T *d) const { d[0] = gather(plane); }
  __device__ inline T combine(const T *d) const { return d[0]; }
  // (interface of the four-corner taps; a single corner has no rows to skip or pair)
  __device__ inline bool row_in_use(int) const { return off >= 0; }
  __device__ inline bool pairable() const { return false; }
  __device__ inline void load_rows(plane_buf_t plane, T *d, bool, bool, bool) const {
    load(plane, d);
  }
  template <bool PAIRS>
  __device__ inline void load_flat(plane_buf_t plane, T *d) const {
    load(plane, d);
  }
  __device__ inline void scatter(T *plane, T v) const {
    if (off >= 0) atomic_add(plane + off, v);
  }
  static constexpr int kCorners = 1;
  __device__ inline int corner_off(int) const { return off; }
  __device__ inline void set_corner_off(int, int v) { off = v; }
  __device__ inline T corner_wt(int) const { return T(1); }
};

// Bilinear (zero padding on both axes) and bispherical (x wraps, y zero-padded).
// Weight products are formed as (A*B), (A*C), (D*B), (D*C) and then multiplied by
// the data, summed left to right: include/core/interpolation.h:22-32.
template <typename T, int MODE>
struct Tap {
  int off[4];
  T wt[4];
  // The two corners of a row are neighbours in memory (x2 == x1 + 1, both inside the plane)
  // or both outside: one load of two elements can fetch them.  False next to the left and
  // right border and at the seam of a wrapped column index.
  bool pair_ok;
  __device__ inline void set(T x, T y, int h, int w) {
    const T x1f = mcx_floor(x), y1f = mcx_floor(y);
    const T x2f = x1f + T(1), y2f = y1f + T(1);
    int x1 = to_int(x1f), y1 = to_int(y1f);
    int x2 = x1 + 1, y2 = y1 + 1;
    bool x1ok, x2ok;
    if (MODE == kInterpBispherical) {
      x1 = wrap_index(x1, w);
      x2 = wrap_index(x2, w);
      x1ok = x2ok = true;
    } else {
      x1ok = x1 >= 0 && x1 <= w - 1;
      x2ok = x2 >= 0 && x2 <= w - 1;
    }
    const bool y1ok = y1 >= 0 && y1 <= h - 1;
    const bool y2ok = y2 >= 0 && y2 <= h - 1;
    pair_ok = (x1ok && x2ok && x2 == x1 + 1) || (!x1ok && !x2ok);
    const T A = y2f - y, B = x2f - x, C = x - x1f, D = y - y1f;
    wt[0] = A * B;
    wt[1] = A * C;
    wt[2] = D * B;
    wt[3] = D * C;
    // A corner of weight exactly zero (integral coordinates) is treated like one outside
    // the plane: it adds 0 to any finite value, and its load or atomic is saved.
    off[0] = (x1ok && y1ok && wt[0] != T(0)) ? y1 * w + x1 : -1;
    off[1] = (x2ok && y1ok && wt[1] != T(0)) ? y1 * w + x2 : -1;
    off[2] = (x1ok && y2ok && wt[2] != T(0)) ? y2 * w + x1 : -1;
    off[3] = (x2ok && y2ok && wt[3] != T(0)) ? y2 * w + x2 : -1;
  }
  template <typename TD>
  __device__ inline T gather(const TD *plane) const {
    T d[4];
#pragma unroll
    for (int i = 0; i < 4; i++) d[i] = (T)load_elem(plane, off[i]);
#pragma unroll
    for (int i = 0; i < 4; i++) d[i] = off[i] >= 0 ? d[i] : T(0);
    return wt[0] * d[0] + wt[1] * d[1] + wt[2] * d[2] + wt[3] * d[3];
  }
  __device__ inline void load(plane_buf_t plane, T *d) const {
#pragma unroll
    for (int i = 0; i < 4; i++)
      d[i] = buf_load(plane, off[i] < 0 ? kOobOffset : (unsigned)off[i] * (unsigned)sizeof(T), T());
  }
  __device__ inline T combine(const T *d) const {
    return wt[0] * d[0] + wt[1] * d[1] + wt[2] * d[2] + wt[3] * d[3];
  }
  // Row r (0: y1, 1: y2) holds a corner that is inside the plane and weighs something.
  __device__ inline bool row_in_use(int r) const { return off[2 * r] >= 0 || off[2 * r + 1] >= 0; }
  __device__ inline bool pairable() const { return pair_ok; }
  // load() with three wave-uniform switches: rows no lane of the wave uses are not loaded
  // at all, and when every lane's tap is pairable a row is one two-element load (its second
  // element then is real data even where its weight is exactly zero, as in the reference's
  // own arithmetic).  The texture addresser, which bounds these gathers, sees a quarter to a
  // half of the instructions.
  __device__ inline void load_rows(plane_buf_t plane, T *d, bool row0, bool row1,
                                   bool pairs) const {
    const bool rows[2] = {row0, row1};
#pragma unroll
    for (int r = 0; r < 2; r++) {
      if (!rows[r]) {
        d[2 * r] = d[2 * r + 1] = T(0);
      } else if (pairs) {
        const auto v = buf_load_pair(
            plane, off[2 * r] < 0 ? kOobOffset : (unsigned)off[2 * r] * (unsigned)sizeof(T), T());
        d[2 * r] = v.x;
        d[2 * r + 1] = v.y;
      } else {
#pragma unroll
        for (int i = 2 * r; i < 2 * r + 2; i++)
          d[i] = buf_load(plane, off[i] < 0 ? kOobOffset : (unsigned)off[i] * (unsigned)sizeof(T),
                          T());
      }
    }
  }
  // load_rows() without its switches: both rows, as two two-element loads (PAIRS; every
  // lane's tap must be pairable) or four single ones.  No branch, so a caller can keep the
  // loads of several planes in flight and the compiler can count them.
  template <bool PAIRS>
  __device__ inline void load_flat(plane_buf_t plane, T *d) const {
    if constexpr (PAIRS) {
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const auto v = buf_load_pair(
            plane, off[2 * r] < 0 ? kOobOffset : (unsigned)off[2 * r] * (unsigned)sizeof(T), T());
        d[2 * r] = v.x;
        d[2 * r + 1] = v.y;
      }
    } else {
      load(plane, d);
    }
  }
  __device__ inline T gather(plane_buf_t plane) const {
    T d[4];
    load(plane, d);
    return combine(d);
  }
  __device__ inline void scatter(T *plane, T v) const {
#pragma unroll
    for (int i = 0; i < 4; i++)
      if (off[i] >= 0) atomic_add(plane + off[i], wt[i] * v);
  }
  static constexpr int kCorners = 4;
  __device__ inline int corner_off(int i) const { return off[i]; }
  __device__ inline void set_corner_off(int i, int v) { off[i] = v; }
  __device__ inline T corner_wt(int i) const { return wt[i]; }
};

// ---- launch helpers ---------------------------------------------------------

inline unsigned div_up(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }

// Dispatch a functor templated on the interpolation mode.
#define MCX_DISPATCH_MODE(interp, ...)                                   \
  switch (mcx::canonical_interp(interp)) {                               \
    case mcx::kInterpBilinear: { constexpr int MODE = mcx::kInterpBilinear; __VA_ARGS__; } break; \
    case mcx::kInterpBispherical: { constexpr int MODE = mcx::kInterpBispherical; __VA_ARGS__; } break; \
    default: { constexpr int MODE = mcx::kInterpNearest; __VA_ARGS__; } break; \
  }

}  // namespace mcx
