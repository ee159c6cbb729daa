// fp32 matrix-core kernels of the mapped convolution for gfx950.
//
// gather_product (convolution forward, transposed-convolution backward-input):
//   y[b,o,n] = bias[o] + sum_{g,k} W[o,g,k] * sample(src[b,g], map[n,k])
// is computed as an implicit GEMM.  A workgroup owns a 2-D tile of 128 output
// pixels and 64 output channels.  The reduction runs tap-major: for each tap k the
// tile's sample locations are resolved once to (offset, weight) pairs held in
// registers, then for each chunk of 16 source channels every thread gathers and
// interpolates 8 samples straight into an LDS tile S[16][128]; the matching slice of
// the (pre-packed) weights goes to LDS as Wt[16][64]; four wavefronts multiply them
// with v_mfma_f32_32x32x2_f32 (each wave: 32 pixels x 64 channels).  Loads for chunk
// t+1 are issued before the MFMAs of chunk t.  No column buffer ever reaches HBM.
#include "mcx_conv.h"
#include "mcx_taps.h"

namespace mcx {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kTilePx = 128;  // output pixels per workgroup
constexpr int kGC = 16;       // source channels per reduction chunk
constexpr int kOT = 64;       // output channels per workgroup
constexpr int kWtLd = kOT + 4;

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD one contiguous
// run of tiles so that neighbouring tiles (which share source rows) share an L2.
__device__ inline int xcd_contiguous_tile(int wg, int total) {
  const int q = total >> 3, r = total & 7;
  const int xcd = wg & 7, slot = wg >> 3;
  return xcd * q + min(xcd, r) + slot;
}

// Repack W[o][g][k] -> Wp[k][g][o] with g padded to 16 and o padded to 64 (zeros),
// so that a reduction chunk's weights are 16 rows of contiguous floats.
__global__ void pack_weights_kernel(const float *__restrict__ w, float *__restrict__ wp, int O,
                                    int G, int K, int Opad, int Gpad) {
  const int64_t total = (int64_t)K * Gpad * Opad;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int o = (int)(e % Opad);
    const int g = (int)((e / Opad) % Gpad);
    const int k = (int)(e / ((int64_t)Opad * Gpad));
    wp[e] = (o < O && g < G) ? w[((int64_t)o * G + g) * K + k] : 0.f;
  }
}

template <int NCORN, int NP>
__global__ __launch_bounds__(kThreads, 2) void gather_product_mfma_kernel(
    const float *__restrict__ src, const float *__restrict__ map, const float *__restrict__ iw,
    const float *__restrict__ wp, const float *__restrict__ bias, float *__restrict__ y, int G,
    int O, int Opad, int Gpad, int SH, int SW, int OH, int OW, int K, int weighted, int wrap,
    int tiles_x, int tiles_per_img, int tw_shift) {
  __shared__ __attribute__((aligned(16))) float S[2][kGC][kTilePx];
  __shared__ __attribute__((aligned(16))) float Wt[2][kGC][kWtLd];

  const int tid = threadIdx.x;
  const int tile = xcd_contiguous_tile(blockIdx.x, gridDim.x);
  const int b = tile / tiles_per_img;
  const int t_in = tile - b * tiles_per_img;
  const int tile_y = t_in / tiles_x, tile_x = t_in - tile_y * tiles_x;
  const int tw_mask = (1 << tw_shift) - 1;
  const int th = kTilePx >> tw_shift;
  const int o0 = blockIdx.y * kOT;
  const int N = OH * OW;
  const int64_t plane = (int64_t)SH * SW;

  // gather role: pixel p of the tile, channels [half*8, half*8+8) of each chunk
  const int p = tid & (kTilePx - 1);
  const int half = tid >> 7;
  const int gi = tile_y * th + (p >> tw_shift), gj = (tile_x << tw_shift) + (p & tw_mask);
  const bool live = gi < OH && gj < OW;
  const int64_t n_g = live ? (int64_t)gi * OW + gj : 0;

  const float *src_b = src + (int64_t)b * G * plane;
  const int chunks = Gpad / kGC;
  const int iters = K * chunks;

  PairTap<NCORN> taps[NP];
  float mx[NP], my[NP], mw[NP];
  float v[8][NP * NCORN];
  float4 wv;

  auto load_map = [&](int k) {
#pragma unroll
    for (int sp = 0; sp < NP; sp++) {
      const int64_t e = (n_g * K + k) * NP + sp;
      mx[sp] = map[e * 2];
      my[sp] = map[e * 2 + 1];
      mw[sp] = weighted ? iw[e] : 1.f;
    }
  };
  auto resolve = [&]() {
#pragma unroll
    for (int sp = 0; sp < NP; sp++)
      resolve_pairs<NCORN>(mx[sp], my[sp], SH, SW, wrap != 0, live ? mw[sp] : 0.f, taps[sp]);
  };
  auto issue = [&](int k, int c) {
    const int g0 = c * kGC + half * 8;
#pragma unroll
    for (int ch = 0; ch < 8; ch++) {
      const int g = min(g0 + ch, G - 1);  // padded channels read a valid plane, weights are 0
      const float *pl = src_b + (int64_t)g * plane;
#pragma unroll
      for (int sp = 0; sp < NP; sp++)
#pragma unroll
        for (int i = 0; i < NCORN; i++) v[ch][sp * NCORN + i] = pl[taps[sp].off[i]];
    }
    // weights of this chunk: 16 rows x 64 floats, one float4 per thread
    const int cc = tid >> 4, o4 = (tid & 15) * 4;
    wv = *reinterpret_cast<const float4 *>(wp + ((int64_t)k * Gpad + c * kGC + cc) * Opad + o0 + o4);
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int ch = 0; ch < 8; ch++) {
      float acc = 0.f;
#pragma unroll
      for (int sp = 0; sp < NP; sp++)
#pragma unroll
        for (int i = 0; i < NCORN; i++)
          acc = __builtin_fmaf(taps[sp].wt[i], v[ch][sp * NCORN + i], acc);
      S[buf][half * 8 + ch][p] = acc;
    }
    const int cc = tid >> 4, o4 = (tid & 15) * 4;
    *reinterpret_cast<float4 *>(&Wt[buf][cc][o4]) = wv;
  };

  floatx16 acc0 = {0}, acc1 = {0};
  const int lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, lhi = lane >> 5;

  load_map(0);
  resolve();
  if (K > 1) load_map(1);
  issue(0, 0);
  int k = 0, c = 0;
  for (int it = 0; it < iters; ++it) {
    const int buf = it & 1;
    stage(buf);
    __syncthreads();
    // advance to the next (tap, chunk) and put its loads in flight
    if (++c == chunks) {
      c = 0;
      ++k;
      if (k < K) {
        resolve();  // from the map values fetched one tap ahead
        if (k + 1 < K) load_map(k + 1);
      }
    }
    if (it + 1 < iters) issue(k, c);
#pragma unroll
    for (int s = 0; s < kGC / 2; s++) {
      const int kk = 2 * s + lhi;
      const float bv = S[buf][kk][wave * 32 + l31];
      const float a0 = Wt[buf][kk][l31];
      const float a1 = Wt[buf][kk][32 + l31];
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, bv, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, bv, acc1, 0, 0, 0);
    }
  }

  // epilogue: lane holds pixel (wave*32 + l31) and 2 x 16 output channels
  const int pe = wave * 32 + l31;
  const int ei = tile_y * th + (pe >> tw_shift), ej = (tile_x << tw_shift) + (pe & tw_mask);
  if (ei < OH && ej < OW) {
    float *yb = y + (int64_t)b * O * N + (int64_t)ei * OW + ej;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int o = o0 + (i >> 2) * 8 + lhi * 4 + (i & 3);
      if (o < O) yb[(int64_t)o * N] = acc0[i] + (bias ? bias[o] : 0.f);
      if (o + 32 < O) yb[(int64_t)(o + 32) * N] = acc1[i] + (bias ? bias[o + 32] : 0.f);
    }
  }
}

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

}  // namespace

size_t mfma_f32_packed_weight_bytes(int64_t O, int64_t G, int64_t K) {
  return (size_t)(K * round_up(G, kGC) * round_up(O, kOT)) * sizeof(float);
}

bool mfma_f32_gather_product_supported(int64_t P) { return P >= 0 && P <= 4; }

// wp: scratch of mfma_f32_packed_weight_bytes(O, G, K) bytes.
int mfma_f32_gather_product(const float *src, const float *map, const float *iw, const float *w,
                            const float *bias, float *y, float *wp, int64_t B, int64_t G,
                            int64_t O, int64_t SH, int64_t SW, int64_t OH, int64_t OW, int64_t K,
                            int64_t P, int interp, hipStream_t s) {
  const int Opad = (int)round_up(O, kOT), Gpad = (int)round_up(G, kGC);
  const int64_t packed = (int64_t)K * Gpad * Opad;
  hipLaunchKernelGGL(pack_weights_kernel, dim3((unsigned)std::min<int64_t>((packed + 255) / 256, 4096)),
                     dim3(256), 0, s, w, wp, (int)O, (int)G, (int)K, Opad, Gpad);
  MCX_HIP_CHECK_LAUNCH();
  // 2-D pixel tiles: 4 x 32 when the output has at least 4 rows, else 1 x 128
  const int tw_shift = OH >= 4 ? 5 : 7;
  const int tw = 1 << tw_shift, th = kTilePx >> tw_shift;
  const int tiles_x = (int)((OW + tw - 1) / tw), tiles_y = (int)((OH + th - 1) / th);
  const int tiles_per_img = tiles_x * tiles_y;
  const int64_t total = (int64_t)tiles_per_img * B;
  if (total > 0x7fffffffLL) return MCX_E_SHAPE;
  dim3 grid((unsigned)total, (unsigned)(Opad / kOT));
  const int mode = canonical_interp(interp);
  const int weighted = P > 0 ? 1 : 0, wrap = mode == kInterpBispherical ? 1 : 0;
  const int np = P > 0 ? (int)P : 1;
#define MCX_LAUNCH(NCORN, NP)                                                                    \
  hipLaunchKernelGGL((gather_product_mfma_kernel<NCORN, NP>), grid, dim3(kThreads), 0, s, src,   \
                     map, iw, wp, bias, y, (int)G, (int)O, Opad, Gpad, (int)SH, (int)SW,         \
                     (int)OH, (int)OW, (int)K, weighted, wrap, tiles_x, tiles_per_img, tw_shift)
  if (mode == kInterpNearest) {
    switch (np) {
      case 1: MCX_LAUNCH(1, 1); break;
      case 2: MCX_LAUNCH(1, 2); break;
      case 3: MCX_LAUNCH(1, 3); break;
      default: MCX_LAUNCH(1, 4); break;
    }
  } else {
    switch (np) {
      case 1: MCX_LAUNCH(4, 1); break;
      case 2: MCX_LAUNCH(4, 2); break;
      case 3: MCX_LAUNCH(4, 3); break;
      default: MCX_LAUNCH(4, 4); break;
    }
  }
#undef MCX_LAUNCH
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

}  // namespace mcx
