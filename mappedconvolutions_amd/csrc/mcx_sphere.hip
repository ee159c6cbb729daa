// Planar-convolution operator on a triangle mesh of the sphere: for every sample direction
// (longitude, latitude) the mesh face its ray pierces, that face's three vertex indices and the
// barycentric weights of the pierced point - the [., K, 3] index and weight maps a weighted
// mapped convolution over mesh vertices is driven by.  Per-face test and output order follow
// the reference's Sphere::_isPointInFace and getPlanarConvolutionOperatorFromSamples
// (ext_modules/src/util/cpp/sphere.cpp:1055-1105, 1117-1270); the search does not: the
// reference walks a breadth-first search over a hierarchy of its own icospheres, one sample
// per OpenMP iteration, while here the mesh is the caller's (any closed triangle mesh around
// the origin) and every sample checks every face, almost all of them with one dot product
// against the face's bounding cone.
#include "mcx_device.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;
constexpr float kInsideTolerance = -1e-3f;  // sphere.cpp:1104

struct V3 {
  float x, y, z;
};
__device__ inline V3 operator-(V3 a, V3 b) { return V3{a.x - b.x, a.y - b.y, a.z - b.z}; }
__device__ inline V3 operator*(V3 a, float s) { return V3{a.x * s, a.y * s, a.z * s}; }
__device__ inline float dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ inline V3 cross(V3 a, V3 b) {
  return V3{a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ inline V3 normalized(V3 a) {
  const float n = sqrtf(dot(a, a));
  return V3{a.x / n, a.y / n, a.z / n};
}
__device__ inline V3 vertex(const float *__restrict__ v, int64_t i) {
  return V3{v[i * 3], v[i * 3 + 1], v[i * 3 + 2]};
}

// Bounding cone of every face: unit axis (the normalised sum of the vertex directions) and the
// cosine a ray must reach to be able to pass the face test, i.e. the cosine of the widest
// vertex angle, lowered by a margin that covers the test's tolerance of 1e-3 in barycentric
// units (a few thousandths of the cone's own opening).  Degenerate faces get a cone nothing
// enters.
__global__ __launch_bounds__(kThreads) void face_cones_kernel(const float *__restrict__ verts,
                                                              const int64_t *__restrict__ faces,
                                                              float4 *__restrict__ cones, int F,
                                                              int V) {
  const int f = blockIdx.x * kThreads + threadIdx.x;
  if (f >= F) return;
  const int64_t ia = faces[f * 3], ib = faces[f * 3 + 1], ic = faces[f * 3 + 2];
  float4 cone = make_float4(0.f, 0.f, 0.f, 2.f);
  if (ia >= 0 && ia < V && ib >= 0 && ib < V && ic >= 0 && ic < V) {
    const V3 a = normalized(vertex(verts, ia)), b = normalized(vertex(verts, ib)),
             c = normalized(vertex(verts, ic));
    const V3 axis = normalized(V3{a.x + b.x + c.x, a.y + b.y + c.y, a.z + b.z + c.z});
    const float cosr = fminf(dot(axis, a), fminf(dot(axis, b), dot(axis, c)));
    if (cosr == cosr) cone = make_float4(axis.x, axis.y, axis.z, cosr - 0.05f * (1.f - cosr) - 1e-6f);
  }
  cones[f] = cone;
}

// Sphere::_isPointInFace, sphere.cpp:1055-1105: the sample is projected along its ray onto the
// plane of the face and expressed in the face's barycentric coordinates (s: third vertex,
// t: second, u: first).  Returns whether all three reach -1e-3.
__device__ inline bool point_in_face(V3 A, V3 B, V3 C, V3 pt, float &s, float &t, float &u) {
  const V3 normal = normalized(cross(C - B, A - B));  // _computeFaceNormal, sphere.cpp:466-484
  const float d = -dot(normal, A);
  const V3 ray = normalized(pt);
  const float denom = dot(normal, ray);
  if (denom < 0.f) return false;  // a face on the far side
  V3 proj;
  if (denom < 1e-12f) {
    const float dist = dot(normal, pt) + d;
    proj = pt - normal * dist;
  } else {
    const float dist = dot(A, normal) / denom;
    proj = ray * dist;
  }
  const V3 BA = B - A, CA = C - A;
  const V3 N = cross(BA, CA);
  const V3 W = proj - A;
  const float nn = dot(N, N);
  s = dot(cross(BA, W), N) / nn;
  t = dot(cross(W, CA), N) / nn;
  u = 1.f - s - t;
  return s >= kInsideTolerance && t >= kInsideTolerance && u >= kInsideTolerance;
}

// One sample per thread; the cones go through LDS, 256 at a time.  Where several faces pass
// the test (a sample within the tolerance of an edge or on a vertex) the one the sample lies
// deepest inside wins, the lower index on ties.
__global__ __launch_bounds__(kThreads) void planar_operator_kernel(
    const float *__restrict__ samples, const float *__restrict__ verts,
    const int64_t *__restrict__ faces, const float4 *__restrict__ cones,
    int64_t *__restrict__ face_idx, int64_t *__restrict__ vertex_idx, float *__restrict__ weights,
    int64_t N, int F, int nearest) {
  __shared__ float4 tile[kThreads];
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool live = i < N;
  V3 pt{0.f, 0.f, 1.f};
  if (live) {
    // core::SphericalToXYZ, include/core/conversions.h:21-26
    const float lon = samples[i * 2], lat = samples[i * 2 + 1];
    pt = V3{cosf(lat) * sinf(lon), -sinf(lat), cosf(lat) * cosf(lon)};
  }
  const V3 ray = normalized(pt);
  int best = -1;
  float bs = 0.f, bt = 0.f, bu = 0.f, depth = -1.f;
  for (int f0 = 0; f0 < F; f0 += kThreads) {
    __syncthreads();
    tile[threadIdx.x] = f0 + (int)threadIdx.x < F ? cones[f0 + threadIdx.x]
                                                  : make_float4(0.f, 0.f, 0.f, 2.f);
    __syncthreads();
    const int nf = min(kThreads, F - f0);
    for (int j = 0; j < nf; j++) {
      const float4 c = tile[j];
      // (written so that a NaN direction passes no cone: faces with vertex indices out of range
      // carry a cosine of 2, which no finite direction reaches either, so their vertices are
      // never read; a sample with a non-finite coordinate gets face -1)
      if (!(ray.x * c.x + ray.y * c.y + ray.z * c.z >= c.w)) continue;
      const int f = f0 + j;
      float s, t, u;
      if (live && point_in_face(vertex(verts, faces[f * 3]), vertex(verts, faces[f * 3 + 1]),
                                vertex(verts, faces[f * 3 + 2]), pt, s, t, u)) {
        const float dpt = fminf(s, fminf(t, u));
        if (dpt > depth) {
          depth = dpt;
          best = f;
          bs = s; bt = t; bu = u;
        }
      }
    }
  }
  if (!live) return;
  face_idx[i] = best;
  if (best < 0) {  // no face contains the ray: the mesh is not closed around the origin
    for (int q = 0; q < 3; q++) {
      vertex_idx[i * 3 + q] = -1;
      weights[i * 3 + q] = 0.f;
    }
    return;
  }
  // weights (s, t, u) go with the face's vertices in reverse order, sphere.cpp:1196-1214
  vertex_idx[i * 3] = faces[best * 3 + 2];
  vertex_idx[i * 3 + 1] = faces[best * 3 + 1];
  vertex_idx[i * 3 + 2] = faces[best * 3];
  if (nearest) {  // maxOfThreeValues, sphere.cpp:1108-1113: strict maxima, else the first
    int m = 0;
    if (bt > bs && bt > bu) m = 1;
    if (bu > bs && bu > bt) m = 2;
    weights[i * 3] = m == 0 ? 1.f : 0.f;
    weights[i * 3 + 1] = m == 1 ? 1.f : 0.f;
    weights[i * 3 + 2] = m == 2 ? 1.f : 0.f;
  } else {
    weights[i * 3] = bs;
    weights[i * 3 + 1] = bt;
    weights[i * 3 + 2] = bu;
  }
}

}  // namespace
}  // namespace mcx

using namespace mcx;

extern "C" size_t mcx_planar_conv_operator_workspace(int64_t F) {
  return F > 0 && F <= 0x7fffffffLL / 3 ? (size_t)F * sizeof(float4) : 0;
}

extern "C" int mcx_planar_conv_operator(const float *samples, const float *vertices,
                                        const int64_t *faces, int64_t *face_idx,
                                        int64_t *vertex_idx, float *weights, void *workspace,
                                        size_t workspace_bytes, int64_t N, int64_t V, int64_t F,
                                        int nearest, void *stream) {
  if (!samples || !vertices || !faces || !face_idx || !vertex_idx || !weights) return MCX_E_NULL;
  if (N <= 0 || V <= 0 || F <= 0 || V > 0x7fffffffLL / 3 || F > 0x7fffffffLL / 3 ||
      N > (int64_t)0x7fffffff * kThreads)
    return MCX_E_SHAPE;
  if (!workspace || workspace_bytes < (size_t)F * sizeof(float4)) return MCX_E_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  float4 *cones = (float4 *)workspace;
  hipLaunchKernelGGL(face_cones_kernel, dim3(div_up(F, kThreads)), dim3(kThreads), 0, s, vertices,
                     faces, cones, (int)F, (int)V);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(planar_operator_kernel, dim3(div_up(N, kThreads)), dim3(kThreads), 0, s,
                     samples, vertices, faces, cones, face_idx, vertex_idx, weights, N, (int)F,
                     nearest ? 1 : 0);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}
