// Weight-form taps for the matrix-core convolution kernels: a sample location is
// resolved to NCORN (element offset, weight) pairs, and the sample is
// sum_i wt[i] * plane[off[i]].  Corners outside the plane get weight 0 and offset 0
// (a safe address), so the inner loops are branch-free.  interp_weights, when
// present, are folded into the corner weights.  Semantics of each mode:
// include/core/interpolation.h:85-238 of the reference.
#pragma once

#include "mcx_device.h"

namespace mcx {

// Storage types of the convolution data: fp32, or bf16 (converted to fp32 on load,
// rounded to nearest-even on store; all arithmetic and accumulation is fp32).
struct bf16_t {
  uint16_t v;
};
__device__ inline float to_f32(float x) { return x; }
__device__ inline float to_f32(bf16_t x) { return __builtin_bit_cast(float, (uint32_t)x.v << 16); }
template <typename TD>
__device__ inline TD from_f32(float x);
template <>
__device__ inline float from_f32<float>(float x) {
  return x;
}
template <>
__device__ inline bf16_t from_f32<bf16_t>(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t{(uint16_t)0x7fc0};  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return bf16_t{(uint16_t)(u >> 16)};
}

// off[] are BYTE offsets of elements, unsigned, so that a load from a wave-uniform
// plane pointer compiles to "scalar base + 32-bit vector offset".
template <int NCORN>
struct PairTap {
  unsigned off[NCORN];
  float wt[NCORN];
};

template <typename TD>
__device__ inline float load_at(const TD *plane, unsigned byte_off) {
  return to_f32(*reinterpret_cast<const TD *>(reinterpret_cast<const char *>(plane) + byte_off));
}

// NCORN == 1: nearest.  NCORN == 4: bilinear (wrap == false) or bispherical (wrap == true).
// ESZ: bytes per data element.
template <int NCORN, int ESZ>
__device__ inline void resolve_pairs(float x, float y, int h, int w, bool wrap, float scale,
                                     PairTap<NCORN> &t) {
  if (NCORN == 1) {
    const int xi = to_int(round_half_away(x));
    const int yi = to_int(round_half_away(y));
    const bool ok = xi >= 0 && xi <= w - 1 && yi >= 0 && yi <= h - 1;
    t.off[0] = ok ? (unsigned)(yi * w + xi) * (unsigned)ESZ : 0u;
    t.wt[0] = ok ? scale : 0.f;
  } else {
    const float x1f = floorf(x), y1f = floorf(y);
    int x1 = to_int(x1f), y1 = to_int(y1f);
    int x2 = x1 + 1, y2 = y1 + 1;
    bool x1ok, x2ok;
    if (wrap) {
      x1 = wrap_index(x1, w);
      x2 = wrap_index(x2, w);
      x1ok = x2ok = true;
    } else {
      x1ok = x1 >= 0 && x1 <= w - 1;
      x2ok = x2 >= 0 && x2 <= w - 1;
    }
    const bool y1ok = y1 >= 0 && y1 <= h - 1;
    const bool y2ok = y2 >= 0 && y2 <= h - 1;
    const float A = (y1f + 1.f) - y, B = (x1f + 1.f) - x, C = x - x1f, D = y - y1f;
    const bool ok[4] = {x1ok && y1ok, x2ok && y1ok, x1ok && y2ok, x2ok && y2ok};
    const int o[4] = {y1 * w + x1, y1 * w + x2, y2 * w + x1, y2 * w + x2};
    const float wv[4] = {A * B, A * C, D * B, D * C};
#pragma unroll
    for (int i = 0; i < NCORN; i++) {
      t.off[i] = ok[i] ? (unsigned)o[i] * (unsigned)ESZ : 0u;
      t.wt[i] = ok[i] ? wv[i] * scale : 0.f;
    }
  }
}

// Coordinate form of the same taps, for scatters that need the destination row
// and column of every corner (valid bit i of `ok` set when corner i is inside).
template <int NCORN>
struct CoordTap {
  int yy[NCORN], xx[NCORN];
  float wt[NCORN];
  unsigned ok;
};

template <int NCORN>
__device__ inline void resolve_coords(float x, float y, int h, int w, bool wrap, float scale,
                                      CoordTap<NCORN> &t) {
  if (NCORN == 1) {
    const int xi = to_int(round_half_away(x));
    const int yi = to_int(round_half_away(y));
    t.ok = (xi >= 0 && xi <= w - 1 && yi >= 0 && yi <= h - 1) ? 1u : 0u;
    t.yy[0] = yi;
    t.xx[0] = xi;
    t.wt[0] = scale;
  } else {
    const float x1f = floorf(x), y1f = floorf(y);
    int x1 = to_int(x1f), y1 = to_int(y1f);
    int x2 = x1 + 1, y2 = y1 + 1;
    bool x1ok, x2ok;
    if (wrap) {
      x1 = wrap_index(x1, w);
      x2 = wrap_index(x2, w);
      x1ok = x2ok = true;
    } else {
      x1ok = x1 >= 0 && x1 <= w - 1;
      x2ok = x2 >= 0 && x2 <= w - 1;
    }
    const bool y1ok = y1 >= 0 && y1 <= h - 1;
    const bool y2ok = y2 >= 0 && y2 <= h - 1;
    const float A = (y1f + 1.f) - y, B = (x1f + 1.f) - x, C = x - x1f, D = y - y1f;
    const int ys[4] = {y1, y1, y2, y2};
    const int xs[4] = {x1, x2, x1, x2};
    const float wv[4] = {A * B, A * C, D * B, D * C};
    t.ok = (x1ok && y1ok ? 1u : 0u) | (x2ok && y1ok ? 2u : 0u) | (x1ok && y2ok ? 4u : 0u) |
           (x2ok && y2ok ? 8u : 0u);
#pragma unroll
    for (int i = 0; i < NCORN; i++) {
      t.yy[i] = ys[i];
      t.xx[i] = xs[i];
      t.wt[i] = wv[i] * scale;
    }
  }
}

}  // namespace mcx
