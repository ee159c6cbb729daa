// Sample-map builders and the cube-map -> equirectangular resampler.
//
// The reference builds its sample maps on the host with torch tensor expressions
// (package/layers/util/spherical_projections.py:12-196, conversions.py:6-189,
// grids.py:23-37); here one thread computes one (pixel, tap) entry directly into device
// memory, so a 512 x 1024 x 25 map never crosses the host link.  The maps are evaluated in
// double precision and rounded once to the output's float: each entry is the correctly
// rounded value of the formula the reference evaluates step by step in float.
//
// cube2rect follows include/util/cuda/cube2rect.cuh:16-64 of the reference in the data's
// own precision: the coordinates are computed in the kernel and the sample is taken from
// the face with the nearest / bilinear interpolators of include/core/interpolation.h:85-160.
#include <algorithm>

#include "mcx_device.h"

namespace mcx {
namespace {

constexpr double kPi = 3.14159265358979323846;

// torch.remainder for a positive divisor (spherical_projections.py:147,190).
__device__ inline double py_mod(double a, double b) {
  double r = fmod(a, b);
  if (r < 0) r += b;
  return r;
}

// (lon, lat) -> (x, y) on an H x W equirectangular image: conversions.py:6-17.
__device__ inline void spherical_to_image(double lon, double lat, int H, int W, double &x,
                                          double &y) {
  x = (W / 2.0) * (lon / kPi + 1.0);
  y = ((H - 1) / 2.0) * (-2.0 * lat / kPi + 1.0);
}

// A point (x, y) of the plane tangent to the unit sphere at latitude `lat` (x towards growing
// longitude, y towards growing latitude), carried back onto the sphere: its latitude and
// its longitude relative to the point of tangency.  (0, 0) gives 0 / 0, as the reference's
// expression does; callers set that tap themselves.
__device__ inline void tangent_plane_to_sphere(double x, double y, double lat, double &dlon,
                                               double &lat_out) {
  const double rho = sqrt(x * x + y * y);
  const double nu = atan(rho);
  lat_out = asin(cos(nu) * sin(lat) + y * sin(nu) * cos(lat) / rho);
  dlon = atan2(x * sin(nu), rho * cos(lat) * cos(nu) - y * sin(lat) * sin(nu));
}

// Tap k of a pixel in row i: everything but the pixel's own longitude depends on (i, k)
// alone.  Returns the tap's latitude and its longitude relative to the pixel (spherical
// projections), or its row and column offset (perspective).
__device__ inline void row_tap(int proj, int H, int W, int kh, int kw, int dilation, int i, int k,
                               double &dlon, double &lat_or_row) {
  const int K = kh * kw;
  const int ci = k / kw - kh / 2, cj = k % kw - kw / 2;
  if (proj == MCX_PROJ_PERSPECTIVE) {
    // spherical_projections.py:73-103: the pixel grid itself
    dlon = (double)(cj * dilation);
    lat_or_row = (double)i + (double)(ci * dilation);
    return;
  }
  // equirectangular_meshgrid of spherical_projections.py:106-114: latitude runs from
  // +pi/2 in row 0 to -pi/2 in row H-1, longitude from -pi in steps of 2 pi / W
  const double res_lat = kPi / (H - 1), res_lon = 2.0 * kPi / W;
  const double lat = kPi / 2 - i * res_lat;
  if (proj == MCX_PROJ_GRID) {
    // spherical_projections.py:39-70: lon/lat in radians, neither wrapped nor converted
    dlon = (double)(cj * dilation) * res_lon;
    lat_or_row = (double)(ci * dilation) * res_lat + lat;
    return;
  }
  const double x = cj * res_lon, y = ci * res_lat;
  if (proj == MCX_PROJ_EQUIRECTANGULAR) {
    // spherical_projections.py:117-150
    lat_or_row = y + lat;
    dlon = x / cos(lat_or_row);
  } else if (k == K / 2) {
    // inverse gnomonic projection about the pixel: spherical_projections.py:153-193; the
    // tap of index K / 2 is set to the pixel itself, every other tap follows the formula
    // (0 / 0 where its offset is zero, as in the reference)
    lat_or_row = lat;
    dlon = 0.0;
  } else {
    tangent_plane_to_sphere(x, y, lat, dlon, lat_or_row);
  }
}

// Gnomonic kernels about arbitrary points of the sphere (the vertices of a mesh):
// package/layers/util/icosphere_functions.py:135-183.  out[v][k] = (lon, lat) of tap k =
// (k / kw - kh / 2, k % kw - kw / 2) x (res_lat, res_lon) on the plane tangent at
// centres[v] = (lon, lat); the tap of index (kh / 2) * kw + kw / 2 is the centre itself;
// longitudes wrapped into [-pi, pi).  Evaluated in double, rounded once.
__global__ void gnomonic_samples_kernel(const float *__restrict__ centres, float *__restrict__ out,
                                        int kh, int kw, double res_lat, double res_lon,
                                        int64_t total) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int K = kh * kw;
  const int k = (int)(e % K);
  const int64_t v = e / K;
  const double lon = centres[v * 2], lat = centres[v * 2 + 1];
  double dlon = 0.0, lat_out = lat;
  if (k != (kh / 2) * kw + kw / 2)
    tangent_plane_to_sphere((k % kw - kw / 2) * res_lon, (k / kw - kh / 2) * res_lat, lat, dlon,
                            lat_out);
  reinterpret_cast<float2 *>(out)[e] =
      make_float2((float)(py_mod(lon + dlon + kPi, 2.0 * kPi) - kPi), (float)lat_out);
}

// out[oi][oj][k] = (x, y); pixel (oi*stride, oj*stride) of the H x W grid, tap k = (k / kw,
// k % kw) with offsets (k / kw - kh / 2, k % kw - kw / 2).  One workgroup writes a run of
// columns of one output row: it first fills an LDS table of the row's K taps (all the
// trigonometry), then every thread combines table entries with its pixel's longitude.
constexpr int kRowTaps = 1024;  // table entries; larger kernels are evaluated per entry

__global__ __launch_bounds__(256) void projection_map_kernel(float *__restrict__ out, int H, int W,
                                                             int kh, int kw, int proj, int stride,
                                                             int dilation, int OW, int cols) {
  __shared__ double2 table[kRowTaps];
  const int K = kh * kw;
  const int oi = blockIdx.y, i = oi * stride;
  const bool tabled = K <= kRowTaps;
  if (tabled) {
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
      double dlon, lat;
      row_tap(proj, H, W, kh, kw, dilation, i, k, dlon, lat);
      table[k] = make_double2(dlon, lat);
    }
    __syncthreads();
  }
  const int oj0 = blockIdx.x * cols, oj1 = min(oj0 + cols, OW);
  const double res_lon = 2.0 * kPi / W;
  float2 *row = reinterpret_cast<float2 *>(out) + (int64_t)oi * OW * K;
  for (int64_t e = (int64_t)oj0 * K + threadIdx.x; e < (int64_t)oj1 * K; e += blockDim.x) {
    const int k = (int)(e % K), j = (int)(e / K) * stride;
    double dlon, lat;
    if (tabled) {
      const double2 t = table[k];
      dlon = t.x;
      lat = t.y;
    } else {
      row_tap(proj, H, W, kh, kw, dilation, i, k, dlon, lat);
    }
    double ox, oy;
    if (proj == MCX_PROJ_PERSPECTIVE) {
      ox = (double)j + dlon;
      oy = lat;
    } else {
      const double lon = -kPi + j * res_lon;
      if (proj == MCX_PROJ_GRID) {
        ox = dlon + lon;
        oy = lat;
      } else {
        // gnomonic adds the pixel's longitude last, the equirectangular form first
        // (spherical_projections.py:144,181): the sum is the same
        const double out_lon = py_mod(lon + dlon + kPi, 2.0 * kPi) - kPi;
        spherical_to_image(out_lon, lat, H, W, ox, oy);
      }
    }
    row[e] = make_float2((float)ox, (float)oy);
  }
}

// 3-D direction -> (face, u, v) with u, v in [0, 1]; faces ordered [-z, -x, +z, +x, +y, -y].
// The six tests are applied in the order of conversions.py:64-111 (the same as
// include/core/conversions.h:75-137) and a later match overrides an earlier one.
template <typename T>
__device__ inline void xyz_to_cube(T x, T y, T z, int &face, T &u, T &v) {
  const T ax = mcx_abs(x), ay = mcx_abs(y), az = mcx_abs(z);
  const bool xp = x > 0, yp = y > 0, zp = z > 0;
  T m = T(1), uc = T(-1), vc = T(-1);  // no match (NaN input): u = v = 0 on face 0
  face = 0;
  if (xp && ax >= ay && ax >= az) { m = ax; uc = -z; vc = -y; face = 3; }
  if (!xp && ax >= ay && ax >= az) { m = ax; uc = z; vc = -y; face = 1; }
  if (yp && ay >= ax && ay >= az) { m = ay; uc = x; vc = z; face = 4; }
  if (!yp && ay >= ax && ay >= az) { m = ay; uc = x; vc = -z; face = 5; }
  if (zp && az >= ax && az >= ay) { m = az; uc = x; vc = -y; face = 2; }
  if (!zp && az >= ax && az >= ay) { m = az; uc = -x; vc = -y; face = 0; }
  u = T(0.5) * (uc / m + T(1));
  v = T(0.5) * (vc / m + T(1));
}

// Map of get_reverse_cube_projection_map (spherical_projections.py:26-30, 261-301): every
// pixel of the dim x 6*dim cube-map image goes to the sphere (pixel centres at +0.5:
// conversions.py:123-181), the tap offset is added in (lon, lat), and the result goes back
// to image coordinates x = face * dim + u, y = v (spherical_projections.py:304-311).
__global__ void cube_projection_map_kernel(float *__restrict__ out, int dim, int kh, int kw,
                                           int stride, int OW, int64_t total) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int K = kh * kw;
  const int k = (int)(e % K);
  const int64_t px = e / K;
  const int i = (int)(px / OW) * stride, j = (int)(px % OW) * stride;
  const int ci = k / kw - kh / 2, cj = k % kw - kw / 2;
  const int face = j / dim;
  const double u = 2.0 * ((j % dim + 0.5) / dim) - 1.0, v = 2.0 * ((i + 0.5) / dim) - 1.0;
  double x, y, z;
  switch (face) {
    case 0: x = -u; y = -v; z = -1.0; break;
    case 1: x = -1.0; y = -v; z = u; break;
    case 2: x = u; y = -v; z = 1.0; break;
    case 3: x = 1.0; y = -v; z = -u; break;
    case 4: x = u; y = 1.0; z = v; break;
    default: x = u; y = -1.0; z = -v; break;
  }
  const double res = kPi / (2.0 * dim);  // grids.py:23-25
  const double lat = atan2(-y, sqrt(x * x + z * z)) + ci * res;  // conversions.py:20-31
  const double lon = atan2(x, z) + cj * res;
  const double dx = cos(lat) * sin(lon), dy = -sin(lat), dz = cos(lat) * cos(lon);
  int f;
  double uu, vv;
  xyz_to_cube(dx, dy, dz, f, uu, vv);
  reinterpret_cast<float2 *>(out)[e] =
      make_float2((float)((double)f * dim + uu * dim), (float)(vv * dim));
}

// One thread per output pixel and group of kCubeChannels channels, which share the
// pixel's face coordinates.
constexpr int kCubeChannels = 16;

// BILINEAR is a template parameter and every load unconditional (a corner outside the image
// reads element 0 and is replaced by zero afterwards), four channels at a time: with the loads
// behind per-lane tests and a run-time corner count each one was waited for on its own
// (bilinear 0.158 ms for 64 channels onto 512 x 1024).
template <typename T, bool BILINEAR>
__global__ void cube2rect_kernel(const T *__restrict__ cube, T *__restrict__ rect, int C, int dim,
                                 int RH, int RW) {
  const int64_t px = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (px >= (int64_t)RH * RW) return;
  const int xr = (int)(px % RW), yr = (int)(px / RW);
  // include/core/conversions.h:27-38: evaluated in double, rounded to T
  // (differences in T, products and quotients in double)
  const T lon = (T)(2 * kPi * (double)((T)xr - (T)RW / 2) / (double)(T)RW);
  const T lat = (T)(kPi * (double)((T)yr - ((T)RH - 1) / 2) / (double)((T)RH - 1));
  T x, y, z;
  if constexpr (sizeof(T) == 4) {
    x = cosf(lat) * sinf(lon);
    y = -sinf(lat);
    z = cosf(lat) * cosf(lon);
  } else {
    x = cos(lat) * sin(lon);
    y = -sin(lat);
    z = cos(lat) * cos(lon);
  }
  int face;
  T u, v;
  xyz_to_cube(x, y, z, face, u, v);
  u *= (T)(dim - 1);
  v *= (T)(dim - 1);
  // The face is addressed inside the dim x 6*dim image: bounds are those of the image
  // from the face's first column on (cube2rect.cuh:47-61), so the right-hand neighbour of
  // a face's last column is the next face's first (its weight is zero there).
  const int width = 6 * dim;
  const int64_t plane = (int64_t)dim * width, start = (int64_t)face * dim;
  const int64_t limit = (int64_t)C * plane;  // elements in the whole cube map
  constexpr int NQ = BILINEAR ? 4 : 1;
  int64_t off[NQ];
  T wt[NQ];
  if constexpr (BILINEAR) {
    const T x1f = mcx_floor(u), y1f = mcx_floor(v);
    const int x1 = to_int(x1f), y1 = to_int(y1f), x2 = x1 + 1, y2 = y1 + 1;
    const bool x1ok = x1 >= 0 && x1 <= width - 1, x2ok = x2 >= 0 && x2 <= width - 1;
    const bool y1ok = y1 >= 0 && y1 <= dim - 1, y2ok = y2 >= 0 && y2 <= dim - 1;
    const T A = (y1f + T(1)) - v, B = (x1f + T(1)) - u, Cw = u - x1f, D = v - y1f;
    wt[0] = A * B; wt[1] = A * Cw; wt[2] = D * B; wt[3] = D * Cw;
    off[0] = x1ok && y1ok ? start + (int64_t)y1 * width + x1 : -1;
    off[1] = x2ok && y1ok ? start + (int64_t)y1 * width + x2 : -1;
    off[2] = x1ok && y2ok ? start + (int64_t)y2 * width + x1 : -1;
    off[3] = x2ok && y2ok ? start + (int64_t)y2 * width + x2 : -1;
  } else {
    const int xi = to_int(round_half_away(u)), yi = to_int(round_half_away(v));
    const bool ok = xi >= 0 && xi <= width - 1 && yi >= 0 && yi <= dim - 1;
    wt[0] = T(1);
    off[0] = ok ? start + (int64_t)yi * width + xi : -1;
  }
  const int c0 = blockIdx.y * kCubeChannels, c1 = min(c0 + kCubeChannels, C);
  constexpr int kStep = 4;
  for (int cb = c0; cb < c1; cb += kStep) {
    T d[kStep][NQ];
    bool ok[kStep][NQ];
#pragma unroll
    for (int i = 0; i < kStep; i++) {
      const int64_t base = (int64_t)min(cb + i, c1 - 1) * plane;
#pragma unroll
      for (int q = 0; q < NQ; q++) {  // never read past the end of the buffer
        ok[i][q] = off[q] >= 0 && base + off[q] < limit;
        d[i][q] = cube[ok[i][q] ? base + off[q] : 0];
      }
    }
#pragma unroll
    for (int i = 0; i < kStep; i++) {
#pragma unroll
      for (int q = 0; q < NQ; q++) d[i][q] = ok[i][q] ? d[i][q] : T(0);
      T r;
      if constexpr (BILINEAR)
        r = wt[0] * d[i][0] + wt[1] * d[i][1] + wt[2] * d[i][2] + wt[3] * d[i][3];
      else
        r = d[i][0];
      if (cb + i < c1) rect[(int64_t)(cb + i) * RH * RW + px] = r;
    }
  }
}

}  // namespace
}  // namespace mcx

extern "C" {

int mcx_projection_map(float *out, int64_t H, int64_t W, int64_t kh, int64_t kw, int proj,
                       int64_t stride, int64_t dilation, void *stream) {
  using namespace mcx;
  if (!out) return MCX_E_NULL;
  if (proj < MCX_PROJ_GRID || proj > MCX_PROJ_PERSPECTIVE) return MCX_E_SHAPE;
  if (H < 1 || W < 1 || kh < 1 || kw < 1 || stride < 1 || dilation < 1) return MCX_E_SHAPE;
  // the spherical grids divide by H - 1 (spherical_projections.py:112 raises for H == 1)
  if (proj != MCX_PROJ_PERSPECTIVE && H < 2) return MCX_E_SHAPE;
  if (H > 0x3fffffff || W > 0x3fffffff || kh * kw > 0x7fff || dilation > 0x7fff)
    return MCX_E_SHAPE;
  const int64_t OH = (H + stride - 1) / stride, OW = (W + stride - 1) / stride;
  if (OH > 65535) return MCX_E_SHAPE;
  // about 8192 entries per workgroup
  const int64_t cols = std::max<int64_t>(1, 8192 / (kh * kw));
  hipLaunchKernelGGL(projection_map_kernel, dim3(div_up(OW, cols), (unsigned)OH), dim3(256), 0,
                     (hipStream_t)stream, out, (int)H, (int)W, (int)kh, (int)kw, proj,
                     (int)stride, (int)dilation, (int)OW, (int)cols);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

int mcx_cube_projection_map(float *out, int64_t cube_dim, int64_t kh, int64_t kw, int64_t stride,
                            void *stream) {
  using namespace mcx;
  if (!out) return MCX_E_NULL;
  if (cube_dim < 1 || kh < 1 || kw < 1 || stride < 1) return MCX_E_SHAPE;
  if (cube_dim > 0x0fffffff || kh * kw > 0x7fff) return MCX_E_SHAPE;
  const int64_t OH = (cube_dim + stride - 1) / stride, OW = (6 * cube_dim + stride - 1) / stride;
  const int64_t total = OH * OW * kh * kw;
  hipLaunchKernelGGL(cube_projection_map_kernel, dim3(div_up(total, 256)), dim3(256), 0,
                     (hipStream_t)stream, out, (int)cube_dim, (int)kh, (int)kw, (int)stride,
                     (int)OW, total);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

int mcx_gnomonic_samples(const float *centres, float *out, int64_t V, int64_t kh, int64_t kw,
                         double res_lat, double res_lon, void *stream) {
  using namespace mcx;
  if (!centres || !out) return MCX_E_NULL;
  if (V < 1 || kh < 1 || kw < 1 || kh * kw > 0x7fff || V > 0x7fffffffLL) return MCX_E_SHAPE;
  const int64_t total = V * kh * kw;
  hipLaunchKernelGGL(gnomonic_samples_kernel, dim3(div_up(total, 256)), dim3(256), 0,
                     (hipStream_t)stream, centres, out, (int)kh, (int)kw, res_lat, res_lon, total);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

int mcx_cube2rect(const void *cubemap, void *rect, int64_t C, int64_t cube_dim, int64_t RH,
                  int64_t RW, int interp, int dtype, void *stream) {
  using namespace mcx;
  if (!cubemap || !rect) return MCX_E_NULL;
  if (dtype != MCX_F32 && dtype != MCX_F64) return MCX_E_DTYPE;
  if (C < 1 || cube_dim < 1 || RH < 1 || RW < 1) return MCX_E_SHAPE;
  if (cube_dim > 0x0fffffff || RH > 0x3fffffff || RW > 0x3fffffff || C > 0x7fffffff)
    return MCX_E_SHAPE;
  if (C > 65535LL * kCubeChannels) return MCX_E_SHAPE;
  const dim3 grid(div_up(RH * RW, 256), div_up(C, kCubeChannels));
  const bool bilinear = interp == 1;  // cube2rect.cuh:49-61: everything else is nearest
#define MCX_LAUNCH_C2R(T, BIL)                                                                  \
  hipLaunchKernelGGL((cube2rect_kernel<T, BIL>), grid, dim3(256), 0, (hipStream_t)stream,       \
                     (const T *)cubemap, (T *)rect, (int)C, (int)cube_dim, (int)RH, (int)RW)
  if (dtype == MCX_F32) {
    if (bilinear) MCX_LAUNCH_C2R(float, true); else MCX_LAUNCH_C2R(float, false);
  } else {
    if (bilinear) MCX_LAUNCH_C2R(double, true); else MCX_LAUNCH_C2R(double, false);
  }
#undef MCX_LAUNCH_C2R
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

}  // extern "C"
