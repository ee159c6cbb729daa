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

// One-shot kernel timing (see mcx_profile_dominant_kernel): a pair of caller-owned events
// recorded right before and after the next launch of a gather-product or weight-gradient
// kernel made by the calling thread.
thread_local hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;
inline void profile_begin(hipStream_t s) {
  if (g_prof_start) (void)hipEventRecord(g_prof_start, s);
}
inline void profile_end(hipStream_t s) {
  if (g_prof_stop) (void)hipEventRecord(g_prof_stop, s);
  g_prof_start = g_prof_stop = nullptr;
}


typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kTilePx = 128;  // output pixels per workgroup
constexpr int kGC = 16;       // source channels per reduction chunk
constexpr int kOT = 64;       // output channels per workgroup
constexpr int kWtLd = kOT + 4;
constexpr int kTapCache = 12;  // cached (offset, weight) pairs per tile pixel (12 KB of LDS)

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD one contiguous
// run of tiles so that neighbouring tiles (which share source rows) share an L2.
__device__ inline int xcd_contiguous_tile(int wg, int total) {
  const int q = total >> 3, r = total & 7;
  const int xcd = wg & 7, slot = wg >> 3;
  return xcd * q + min(xcd, r) + slot;
}

// Whether a pair beyond the first two of a tap is in use anywhere in the map, from the pair
// mask: one word (at least 4 then), or `words` words of which any may say so (one per block
// of the launch that examined the map).  Called by whole waves.
__device__ inline bool later_pairs_in_use(const int *__restrict__ mask, int words) {
  if (words <= 1) return (unsigned)*mask >= (1u << 2);
  const int lane = threadIdx.x & 63;
  const unsigned v = (unsigned)mask[lane < words ? lane : 0];
  return __builtin_amdgcn_ballot_w64(v >= (1u << 2)) != 0;
}

// Small jobs that ride on the weight-packing launch (a launch costs 4 to 8 us even when its
// kernel does next to nothing, and small problems are made of launches):
//   * ZeroJob: clear a region of the scratch (counters and flags of a transposed map);
//   * PairMaskJob: the pair mask of a SMALL map, by the launch's last `blocks` (at most 64)
//     blocks, each of which stores the bits it found into a word of its own - no clearing
//     launch before, no atomics; the readers OR the words (later_pairs_in_use).
struct ZeroJob {
  uint4 *ptr;      // 16-byte aligned
  int64_t count;   // 16-byte words
};
struct PairMaskJob {
  const float *map, *iw;
  int *mask;       // `blocks` words; nullptr: no job
  int blocks, np, weighted, wrap, gh, gw, ncorn;
  int64_t total;   // (location, tap) entries
};

// Bits of the (point, corner) pairs with a nonzero weight anywhere among the entries this
// block walks (block `block` of `blocks`); valid in every thread on return.
template <int NCORN>
__device__ inline unsigned block_pair_mask(const float *__restrict__ map,
                                           const float *__restrict__ iw, int np, int weighted,
                                           int wrap, int GH, int GW, int64_t total, int block,
                                           int blocks) {
  __shared__ unsigned block_mask;
  if (threadIdx.x == 0) block_mask = 0;
  __syncthreads();
  unsigned m = 0;
  const int64_t first = (int64_t)block * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)blocks * blockDim.x;
  for (int64_t e = first; e < total; e += stride) {
    for (int sp = 0; sp < np; sp++) {
      const int64_t q = e * np + sp;
      PairTap<NCORN> t;
      resolve_pairs<NCORN, 4>(map[q * 2], map[q * 2 + 1], GH, GW, wrap != 0,
                              weighted ? iw[q] : 1.f, t);
#pragma unroll
      for (int i = 0; i < NCORN; i++)
        if (t.wt[i] != 0.f) m |= 1u << (sp * NCORN + i);
    }
  }
  for (int d = 32; d > 0; d >>= 1) m |= __shfl_xor(m, d);
  if ((threadIdx.x & 63) == 0 && m) atomicOr(&block_mask, m);
  __syncthreads();
  return block_mask;
}

// Repack W[o][g][k] for the matrix-core kernels, with g padded to 16 and o padded to 64
// (zeros); `transposed` reads W[g][o][k] instead (weights stored source-channel major).
//   fp32 storage: Wp[k][g][o] floats, so that a reduction chunk's weights are 16 rows of
//   contiguous floats.
//   bf16 storage feeds v_mfma_f32_32x32x16_bf16: one instruction multiplies a 32 x 16 block of
//   weights by a 16 x 32 block of samples, a lane holding 8 consecutive reduction elements
//   (channels kg*8 .. kg*8+7, kg = lane / 32) of its row or column in 16 bytes.  Weights are
//   therefore packed as Wb[k][chunk][kg][o][8] bf16: the 64 x 16 slice of a (tap, chunk) is two
//   runs of 64 x 16 bytes that are copied linearly into LDS.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// acc + w.lo * word.lo + w.hi * word.hi (v_dot2_f32_bf16: products exact, fp32 sum)
__device__ inline float dot_bf16(unsigned word, unsigned w, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, word),
                                         __builtin_bit_cast(bf16x2, w), acc, false);
}

// w.lo * word.lo + w.hi * word.hi, the head of such a sum.  (Written out because the compiler
// renders dot_bf16(word, w, 0) as the accumulating two-operand form behind a move of zero:
// one instruction in three of an interpolation.)
__device__ inline float dot_bf16_first(unsigned word, unsigned w) {
  float r;
  asm("v_dot2_f32_bf16 %0, %1, %2, 0" : "=v"(r) : "v"(word), "v"(w));
  return r;
}

template <typename TD>
__global__ __launch_bounds__(256) void pack_weights_kernel(
    const TD *__restrict__ w, void *__restrict__ packed_out, int O, int G, int K, int Opad,
    int Gpad, int transposed, int *__restrict__ clear, ZeroJob zero, PairMaskJob pm) {
  if (clear && blockIdx.x == 0 && threadIdx.x == 0) *clear = 0;  // a flag word of the caller
  int blocks = gridDim.x;
  if (pm.mask) {
    blocks -= pm.blocks;
    if ((int)blockIdx.x >= blocks) {  // the last blocks: the map's pair mask, nothing else
      const int mb = (int)blockIdx.x - blocks;
      const unsigned m =
          pm.ncorn == 1 ? block_pair_mask<1>(pm.map, pm.iw, pm.np, pm.weighted, pm.wrap, pm.gh,
                                             pm.gw, pm.total, mb, pm.blocks)
                        : block_pair_mask<4>(pm.map, pm.iw, pm.np, pm.weighted, pm.wrap, pm.gh,
                                             pm.gw, pm.total, mb, pm.blocks);
      if (threadIdx.x == 0) pm.mask[mb] = (int)m;
      return;
    }
  }
  const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)blocks * blockDim.x;
  const int64_t total = (int64_t)K * Gpad * Opad;
  if constexpr (sizeof(TD) == 2) {
    uint16_t *wb = reinterpret_cast<uint16_t *>(packed_out);
    const int chunks = Gpad / kGC;
    for (int64_t e = first; e < total; e += stride) {
      const int j = (int)(e & 7);
      const int o = (int)((e >> 3) % Opad);
      const int kg = (int)((e / ((int64_t)8 * Opad)) & 1);
      const int c = (int)((e / ((int64_t)16 * Opad)) % chunks);
      const int k = (int)(e / ((int64_t)16 * Opad * chunks));
      const int g = c * kGC + kg * 8 + j;
      const int64_t wi = transposed ? ((int64_t)g * O + o) * K + k : ((int64_t)o * G + g) * K + k;
      wb[e] = (o < O && g < G) ? from_f32<bf16_t>(to_f32(w[wi])).v : (uint16_t)0;
    }
  } else {
    float *wp = reinterpret_cast<float *>(packed_out);
    for (int64_t e = first; e < total; e += stride) {
      const int o = (int)(e % Opad);
      const int g = (int)((e / Opad) % Gpad);
      const int k = (int)(e / ((int64_t)Opad * Gpad));
      const int64_t wi = transposed ? ((int64_t)g * O + o) * K + k : ((int64_t)o * G + g) * K + k;
      wp[e] = (o < O && g < G) ? to_f32(w[wi]) : 0.f;
    }
  }
  for (int64_t i = first; i < zero.count; i += stride) zero.ptr[i] = make_uint4(0u, 0u, 0u, 0u);
}

// x[b][g][n] -> xt[b][n][Gpad] (channels past G zero): 64 pixels x 64 channels per
// workgroup through LDS, coalesced on both sides.
template <typename TD>
__global__ __launch_bounds__(256) void to_channel_last_kernel(const TD *__restrict__ x,
                                                              TD *__restrict__ xt, int G, int Gpad,
                                                              int64_t plane) {
  __shared__ TD tile[64][65];
  const int64_t n0 = (int64_t)blockIdx.x * 64;
  const int g0 = blockIdx.y * 64, b = blockIdx.z;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int g = g0 + ly + 4 * r;
    const int64_t n = n0 + lx;
    tile[ly + 4 * r][lx] = (g < G && n < plane) ? x[((int64_t)b * G + g) * plane + n] : TD{};
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int64_t n = n0 + ly + 4 * r;
    const int g = g0 + lx;
    if (n < plane && g < Gpad) xt[((int64_t)b * plane + n) * Gpad + g] = tile[lx][ly + 4 * r];
  }
}

// x[b][g][n] -> xt[b][g/8][n][g%8] (channels past G zero): a thread gathers the 8 channels of
// one pixel (each of the 8 loads is contiguous across the wave) and writes them as one vector.
template <typename TD>
__global__ __launch_bounds__(256) void to_channel_blocks_kernel(const TD *__restrict__ x,
                                                                TD *__restrict__ xt, int G,
                                                                int64_t plane,
                                                                const int *__restrict__ pair_mask) {
  // (with a pair mask: the copy is for a kernel that only runs while the mask is below 4)
  if (pair_mask && (unsigned)*pair_mask >= (1u << 2)) return;
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int g8 = blockIdx.y, b = blockIdx.z;
  if (n >= plane) return;
  struct alignas(8 * sizeof(TD)) Block { TD c[8]; } v;
#pragma unroll
  for (int c = 0; c < 8; c++) {
    const int g = g8 * 8 + c;
    v.c[c] = g < G ? x[((int64_t)b * G + g) * plane + n] : TD{};
  }
  reinterpret_cast<Block *>(xt)[((int64_t)b * gridDim.y + g8) * plane + n] = v;
}

// y[b][a][pixel] -> yt[b][tile][a / 32][mb][s4][lane][8]: the plain operand of a weight gradient
// cut into pixel tiles of 128 (tw_shift: the tile is (128 >> tw_shift) rows of 1 << tw_shift
// pixels; pixels outside the image and channels past A are zeros) and, inside a tile, into the
// MFMA fragments of weight_grad_bf16_ring_kernel: a slab is 32 channels, the rows of one wave;
// fragment (mb, s4) holds, for lane (l15 = lane & 15, lq = lane >> 4), pixels 32 * s4 + 8 * lq
// .. + 7 of channel 16 * mb + l15 of the slab.  A wave of that kernel then loads a fragment as
// one contiguous kilobyte straight into its operand registers.
// One workgroup: one slab of kFragTiles consecutive tiles through LDS (reads: runs of up to a
// kilobyte of a channel's row; writes: each tile's slab, 8 KB, in one piece).  MW is a multiple
// of 8.
constexpr int kFragTiles = 4;
__global__ __launch_bounds__(256) void to_plain_fragments_kernel(const bf16_t *__restrict__ y,
                                                                 bf16_t *__restrict__ yt, int A,
                                                                 int MH, int MW, int tiles_x,
                                                                 int tiles_per_img, int tw_shift) {
  __shared__ __attribute__((aligned(16))) uint16_t T[kFragTiles][32][kTilePx + 8];
  const int slab = blockIdx.y, b = blockIdx.z;
  const int px = (threadIdx.x & 15) * 8;
  const int64_t N = (int64_t)MH * MW;
  uint4 v[kFragTiles][2];
#pragma unroll
  for (int i = 0; i < kFragTiles; i++) {
    const int tile = min((int)blockIdx.x * kFragTiles + i, tiles_per_img - 1);
    const int tile_y = tile / tiles_x, tile_x = tile - tile_y * tiles_x;
    const int si = tile_y * (kTilePx >> tw_shift) + (px >> tw_shift);
    const int sj = (tile_x << tw_shift) + (px & ((1 << tw_shift) - 1));
    const bool inside = si < MH && sj < MW;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int a = slab * 32 + h * 16 + (threadIdx.x >> 4);
      v[i][h] = make_uint4(0u, 0u, 0u, 0u);
      if (inside && a < A)
        v[i][h] = *reinterpret_cast<const uint4 *>(y + ((int64_t)b * A + a) * N +
                                                   (int64_t)si * MW + sj);
    }
  }
#pragma unroll
  for (int i = 0; i < kFragTiles; i++)
#pragma unroll
    for (int h = 0; h < 2; h++)
      *reinterpret_cast<uint4 *>(&T[i][h * 16 + (threadIdx.x >> 4)][px]) = v[i][h];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kFragTiles; i++) {
    const int tile = blockIdx.x * kFragTiles + i;
    if (tile >= tiles_per_img) break;
    uint4 *dst = reinterpret_cast<uint4 *>(yt) +
                 (((int64_t)b * tiles_per_img + tile) * gridDim.y + slab) * 512;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int o = h * 256 + threadIdx.x;  // (mb, s4, lane)
      const int mb = o >> 8, s4 = (o >> 6) & 3, lane = o & 63;
      dst[o] = *reinterpret_cast<const uint4 *>(
          &T[i][mb * 16 + (lane & 15)][32 * s4 + 8 * (lane >> 4)]);
    }
  }
}

// LDS operand tiles of the gather-product kernel, double-buffered.
template <typename TD, int OG>
struct OperandTiles {  // fp32: samples S[chunk channel][pixel], weights Wt[chunk channel][o]
  float S[2][kGC][kTilePx];
  float Wt[2][kGC][kOT * OG + 4];
};
template <int OG>
struct OperandTiles<bf16_t, OG> {  // bf16: 16-byte groups of 8 channels, [kg][pixel] and [kg][o]
  uint4 S[2][2][kTilePx];
  uint4 Wt[2][2][2 * kOT];
};

// OG: groups of 64 output channels per workgroup: 2 where the gather, not the MFMA, bounds the
// kernel and is then shared by twice the outputs (bf16 storage; fp32 over a channel-last
// source, whose every entry is a read of an unrelated record).
// CL: `src` is a channel-last copy [B][SH*SW][Gpad] of the source (made by
// to_channel_last_kernel): a sample's 8 channels are then one or two 16-byte loads from
// one cache line instead of 8 loads from 8 lines.  Used for single-row sources (mesh
// signals), whose maps point anywhere.  With `cl_blocked` the copy is [B][Gpad/8][SH*SW][8]
// (made by to_channel_blocks_kernel): neighbouring pixels stay neighbours, so image-like
// sources keep their coalescing and a sample's 8 channels are still one load; used with bf16
// storage, where the number of load instructions bounds the kernel.
// NA: leading (offset, weight) pairs of a tap that are loaded and added.  NA == NP * NCORN is
// the general form, which skips the pairs a tile's mask shows to be zero across the tile.
// NA == 2 (four-pair taps) is the branch-free form for maps that use nothing but the first
// two pairs anywhere (bilinear with integral rows, transposed maps with at most two
// contributions per cell): both forms are launched and `pair_mask` (at least 4 iff a pair
// beyond the first two is in use somewhere in the map) lets exactly one of them run.
template <typename TD, int NCORN, int NP, int OG, bool CL, int NA>
__global__ __launch_bounds__(kThreads, OG == 1 ? 4 : 3) void gather_product_mfma_kernel(
    const TD *__restrict__ src, const float *__restrict__ map, const float *__restrict__ iw,
    const float *__restrict__ wp, const TD *__restrict__ bias, TD *__restrict__ y, int G,
    int O, int Opad, int Gpad, int SH, int SW, int OH, int OW, int K, int weighted, int wrap,
    int tiles_x, int tiles_per_img, int tw_shift, const int *__restrict__ gate, int run_if_zero,
    const float *__restrict__ addend, const int *__restrict__ pair_mask, int run_if_leading,
    int packed_map, int accumulate, int cl_blocked, const int *__restrict__ row_mask,
    int mask_words) {
  constexpr int NE = NP * NCORN;         // (offset, weight) pairs per pixel and tap
  static_assert(NA >= 1 && NA <= NE, "NA counts leading pairs");
  constexpr bool kMasked = NA == NE;
  // taps cached in LDS at a time: 12 pairs per pixel, or 6 where that leaves room for a
  // fifth workgroup on the CU
  constexpr int kPairs = (NA <= 2 && OG == 1) ? kTapCache / 2 : kTapCache;
  constexpr int TG = NA <= 2 ? kPairs / NA : (kTapCache / NE > 0 ? kTapCache / NE : 1);
  constexpr bool kBf16 = sizeof(TD) == 2;
  __shared__ __attribute__((aligned(16))) OperandTiles<TD, OG> T;
  __shared__ __attribute__((aligned(16))) unsigned TapOff[TG][kTilePx][NA];
  __shared__ __attribute__((aligned(16))) float TapWt[TG][kTilePx][NA];
  // Bit e of TapMask[kl][h]: some pixel of the half-tile resolved by wave pair h has a
  // nonzero weight in pair e of tap kl.  Pairs that are zero across the whole tile
  // (bilinear corners of integral coordinates, unused slots) are neither loaded nor
  // accumulated.
  __shared__ unsigned TapMask[TG][2][2];
  if (gate && ((*gate == 0) != (run_if_zero != 0))) return;  // device-side path selection
  if (pair_mask && !row_mask &&
      (!later_pairs_in_use(pair_mask, mask_words) != (run_if_leading != 0)))
    return;
  // a pass that adds onto y (the second level of a transposed map) has nothing to do when
  // no pair of its map is in use
  if (accumulate && pair_mask && *pair_mask == 0) return;

  const int tid = threadIdx.x;
  const int tile = xcd_contiguous_tile(blockIdx.x, gridDim.x);
  const int b = tile / tiles_per_img;
  const int t_in = tile - b * tiles_per_img;
  const int tile_y = t_in / tiles_x, tile_x = t_in - tile_y * tiles_x;
  const int tw_mask = (1 << tw_shift) - 1;
  const int th = kTilePx >> tw_shift;
  if (pair_mask && row_mask) {
    // The two-pair form serves the whole map when no tap anywhere uses a later pair; with
    // `row_mask` (one word per row of output pixels, nonzero iff a tap of the row does) it
    // serves every tile whose rows are clear, and the general form the others: a few border
    // rows that hold more must not put the whole image on the slower form.
    bool leading = (unsigned)*pair_mask < (1u << 2);
    if (!leading && row_mask) {
      int any = 0;
      for (int r = tile_y * th; r < min(tile_y * th + th, OH); r++) any |= row_mask[r];
      leading = any == 0;
    }
    if (leading != (run_if_leading != 0)) return;
  }
  const int o0 = blockIdx.y * (kOT * OG);
  const int N = OH * OW;
  const int64_t plane = (int64_t)SH * SW;
  const int64_t plane_bytes = plane * (int64_t)sizeof(TD);

  // gather role: pixel p of the tile, channels [half*8, half*8+8) of each chunk
  const int p = tid & (kTilePx - 1);
  const int half = __builtin_amdgcn_readfirstlane(tid >> 7);  // wave-uniform: scalar addressing
  const int gi = tile_y * th + (p >> tw_shift), gj = (tile_x << tw_shift) + (p & tw_mask);
  const bool live = gi < OH && gj < OW;
  const int64_t n_g = live ? (int64_t)gi * OW + gj : 0;

  const TD *src_b = src + (int64_t)b * (CL ? Gpad : G) * plane;
  const int chunks = Gpad / kGC;

  unsigned off[NE];
  float wt[NE];
  float v[8][NE];
  unsigned tmask = 0;
  float4 wv[OG];  // fp32: this thread's share of the next weight chunk
  unsigned wb8[2 * OG];  // bf16: likewise, 8 * OG bytes
  const int w_off = (tid >> 4) * Opad + (tid & 15) * 4;

  auto load_tap = [&](int kl) {  // cached pairs of tap kl of the group -> registers
    if constexpr (kMasked)
      tmask = __builtin_amdgcn_readfirstlane(TapMask[kl][0][0] | TapMask[kl][0][1] |
                                             TapMask[kl][1][0] | TapMask[kl][1][1]);
#pragma unroll
    for (int i = 0; i < NA; i++) {
      off[i] = TapOff[kl][p][i];
      wt[i] = TapWt[kl][p][i];
    }
  };
  // Plane bases of this thread's 8 channels of a chunk (scalar registers); they change
  // only when the chunk does, not with every tap.
  const TD *pl[8];
  auto set_chunk = [&](int c) {
    const int g0 = c * kGC + half * 8;
    if constexpr (CL) {
      // the 8 channels are contiguous; offsets select the pixel
      pl[0] = cl_blocked ? src_b + (int64_t)(g0 >> 3) * plane * 8 : src_b + g0;
    } else if (g0 + 8 <= G) {  // all eight planes exist: one product, then additions
      const char *q = reinterpret_cast<const char *>(src_b) + (int64_t)g0 * plane_bytes;
#pragma unroll
      for (int ch = 0; ch < 8; ch++) {
        pl[ch] = reinterpret_cast<const TD *>(q);
        q += plane_bytes;
      }
    } else {
#pragma unroll
      for (int ch = 0; ch < 8; ch++)  // padded channels read a valid plane, weights are 0
        pl[ch] = src_b + (int64_t)min(g0 + ch, G - 1) * plane;
    }
  };
  auto issue = [&](int k, int c) {
#pragma unroll
    for (int i = 0; i < NA; i++) {
      if (kMasked && !((tmask >> i) & 1u)) continue;  // wave-uniform
      if constexpr (CL) {
        const char *row = reinterpret_cast<const char *>(pl[0]) + off[i];
        if constexpr (kBf16) {
          const uint4 q = *reinterpret_cast<const uint4 *>(row);
          const unsigned w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int j = 0; j < 4; j++) {
            v[2 * j][i] = __builtin_bit_cast(float, w4[j] << 16);
            v[2 * j + 1][i] = __builtin_bit_cast(float, w4[j] & 0xffff0000u);
          }
        } else {
          const float4 q0 = reinterpret_cast<const float4 *>(row)[0];
          const float4 q1 = reinterpret_cast<const float4 *>(row)[1];
          v[0][i] = q0.x; v[1][i] = q0.y; v[2][i] = q0.z; v[3][i] = q0.w;
          v[4][i] = q1.x; v[5][i] = q1.y; v[6][i] = q1.z; v[7][i] = q1.w;
        }
      } else {
#pragma unroll
        for (int ch = 0; ch < 8; ch++) v[ch][i] = load_at(pl[ch], off[i]);
      }
    }
    if constexpr (kBf16) {
      // weights of this chunk: two runs (kg = 0, 1) of 64*OG x 16 bytes, 8*OG bytes per thread
      const char *wchunk = reinterpret_cast<const char *>(wp) +
                           ((((int64_t)k * chunks + c) * 2 + (tid >> 7)) * Opad + o0) * 16;
      if constexpr (OG == 1) {
        const uint2 t2 = *reinterpret_cast<const uint2 *>(wchunk + (tid & 127) * 8);
        wb8[0] = t2.x; wb8[1] = t2.y;
      } else {
        const uint4 t4 = *reinterpret_cast<const uint4 *>(wchunk + (tid & 127) * 16);
        wb8[0] = t4.x; wb8[1] = t4.y; wb8[2 % (2 * OG)] = t4.z; wb8[3 % (2 * OG)] = t4.w;
      }
    } else {
      // weights of this chunk: 16 rows x 64 floats, one float4 per thread
      const float *wchunk = wp + ((int64_t)k * Gpad + c * kGC) * Opad + o0;  // uniform
#pragma unroll
      for (int og = 0; og < OG; og++)
        wv[og] = *reinterpret_cast<const float4 *>(wchunk + w_off + og * kOT);
    }
  };
  auto stage = [&](int buf) {
    float sv[8];
#pragma unroll
    for (int ch = 0; ch < 8; ch++) sv[ch] = 0.f;
#pragma unroll
    for (int i = 0; i < NA; i++) {
      if (kMasked && !((tmask >> i) & 1u)) continue;
#pragma unroll
      for (int ch = 0; ch < 8; ch++) sv[ch] = __builtin_fmaf(wt[i], v[ch][i], sv[ch]);
    }
    if constexpr (kBf16) {
      uint4 q;
      q.x = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{sv[0], sv[1]}, bf16x2));
      q.y = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{sv[2], sv[3]}, bf16x2));
      q.z = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{sv[4], sv[5]}, bf16x2));
      q.w = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{sv[6], sv[7]}, bf16x2));
      T.S[buf][half][p] = q;
      if constexpr (OG == 1)
        reinterpret_cast<uint2 *>(&T.Wt[buf][tid >> 7][0])[tid & 127] = uint2{wb8[0], wb8[1]};
      else
        T.Wt[buf][tid >> 7][tid & 127] =
            uint4{wb8[0], wb8[1], wb8[2 % (2 * OG)], wb8[3 % (2 * OG)]};
    } else {
#pragma unroll
      for (int ch = 0; ch < 8; ch++) T.S[buf][half * 8 + ch][p] = sv[ch];
      const int cc = tid >> 4, o4 = (tid & 15) * 4;
#pragma unroll
      for (int og = 0; og < OG; og++)
        *reinterpret_cast<float4 *>(&T.Wt[buf][cc][og * kOT + o4]) = wv[og];
    }
  };

  floatx16 acc[2 * OG];
#pragma unroll
  for (int m = 0; m < 2 * OG; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[m][i] = 0.f;
  const int lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, lhi = lane >> 5;

  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += TG) {  // tap groups
    const int kn = min(TG, K - k0);
    // Resolve the group's taps once per tile into LDS: thread (p, half) takes every
    // other tap of pixel p.  All channel chunks reuse them.
    __syncthreads();  // the previous group's units are done with the cache and with S/Wt
    if (tid < TG * 4) (&TapMask[0][0][0])[tid] = 0u;  // slots no wave writes below
    __syncthreads();
    for (int kl = half; kl < kn; kl += 2) {
      unsigned m = 0;
      // points whose pairs all lie beyond the leading NA are known to weigh nothing
      constexpr int kPoints = (NA + NCORN - 1) / NCORN;
#pragma unroll
      for (int sp = 0; sp < kPoints; sp++) {
        const int64_t e = (n_g * K + k0 + kl) * NP + sp;
        PairTap<NCORN> t;
        if (NCORN == 1 && packed_map) {
          // pre-resolved entry (a transposed map or a plan's gather part): element index of the
          // source and weight, stored [tap][slot][pixel] so that the lanes of a wave, which
          // hold neighbouring pixels, read neighbouring entries
          const float2 q = reinterpret_cast<const float2 *>(
              map)[((int64_t)(k0 + kl) * NP + sp) * N + n_g];
          t.off[0] = __builtin_bit_cast(unsigned, q.x) * (unsigned)sizeof(TD);
          t.wt[0] = live ? q.y : 0.f;
        } else {
          resolve_pairs<NCORN, sizeof(TD)>(map[e * 2], map[e * 2 + 1], SH, SW, wrap != 0,
                                           live ? (weighted ? iw[e] : 1.f) : 0.f, t);
        }
#pragma unroll
        for (int i = 0; i < NCORN; i++) {
          if (sp * NCORN + i >= NA) continue;
          TapOff[kl][p][sp * NCORN + i] =
              CL ? t.off[i] * (unsigned)(cl_blocked ? 8 : Gpad) : t.off[i];
          TapWt[kl][p][sp * NCORN + i] = t.wt[i];
          if (kMasked && __builtin_amdgcn_ballot_w64(t.wt[i] != 0.f)) m |= 1u << (sp * NCORN + i);
        }
      }
      if (kMasked && (tid & 63) == 0) TapMask[kl][half][(tid >> 6) & 1] = m;
    }
    __syncthreads();

    // Units run chunk-major with the tap fastest: the source rows a 16-channel chunk
    // touches are reused by all taps of the group while they are still in cache.  A
    // channel-last source (a mesh signal: every entry of a tap points at an unrelated vertex,
    // whose channels lie in one record) runs tap-major with the chunk fastest instead, so that
    // a record is used up while its lines are in cache: chunk-major re-read every record once
    // per chunk from memory.
    const bool chunk_fastest = CL && !cl_blocked;
    const int units = chunks * kn;
    if constexpr (CL && kBf16) {
      // bf16 storage, staged source: a unit is NA 16-byte loads per thread and four short
      // MFMAs per wave, far too little work to cover the latency of the next unit's loads.
      // The loads of kDepth units are kept in flight instead (a ring of registers; the unit
      // loop is unrolled by kDepth so that every ring slot has a fixed register).
      constexpr int kDepth = NA <= 2 ? 4 : NA <= 4 ? 2 : 1;
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
      u32x4 ring[kDepth][NA];
      u32x4 wring[kDepth];  // this thread's share of the unit's weights (8 * OG bytes)
      int ki = 0, ci = 0;   // the unit whose loads are issued next
      int ks = 0, cs = 0;   // tap (and, tap-major, chunk) of the unit that is staged next
      // (issued unconditionally, past the last unit too, where it reads the last chunk
      // again: a load that depends on a branch would make every later wait a full one)
      auto issue_slot = [&](int d) {
        const int cc = min(ci, chunks - 1);
        const int g0 = cc * kGC + half * 8;
        const char *base = reinterpret_cast<const char *>(
            cl_blocked ? src_b + (int64_t)(g0 >> 3) * plane * 8 : src_b + g0);
#pragma unroll
        for (int i = 0; i < NA; i++)
          ring[d][i] = *reinterpret_cast<const u32x4 *>(base + TapOff[ki][p][i]);
        const char *wchunk = reinterpret_cast<const char *>(wp) +
                             ((((int64_t)(k0 + ki) * chunks + cc) * 2 + (tid >> 7)) * Opad + o0) * 16;
        if constexpr (OG == 1) {
          const uint2 t2 = *reinterpret_cast<const uint2 *>(wchunk + (tid & 127) * 8);
          wring[d] = u32x4{t2.x, t2.y, 0u, 0u};
        } else {
          wring[d] = *reinterpret_cast<const u32x4 *>(wchunk + (tid & 127) * 16);
        }
        if (chunk_fastest) {
          if (++ci == chunks) {
            ci = 0;
            ki = min(ki + 1, kn - 1);  // (past the last unit: the last tap again)
          }
        } else if (++ki == kn) {
          ki = 0;
          ++ci;
        }
      };
      auto stage_slot = [&](int d, int b) {
        float sv[8];
#pragma unroll
        for (int ch = 0; ch < 8; ch++) sv[ch] = 0.f;
#pragma unroll
        for (int i = 0; i < NA; i++) {
          const float wgt = TapWt[ks][p][i];
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const unsigned w2 = ring[d][i][j];
            sv[2 * j] = __builtin_fmaf(wgt, __builtin_bit_cast(float, w2 << 16), sv[2 * j]);
            sv[2 * j + 1] = __builtin_fmaf(wgt, __builtin_bit_cast(float, w2 & 0xffff0000u),
                                           sv[2 * j + 1]);
          }
        }
        u32x4 q;
#pragma unroll
        for (int j = 0; j < 4; j++)
          q[j] = __builtin_bit_cast(
              unsigned, __builtin_convertvector(floatx2{sv[2 * j], sv[2 * j + 1]}, bf16x2));
        *reinterpret_cast<u32x4 *>(&T.S[b][half][p]) = q;
        if constexpr (OG == 1)
          reinterpret_cast<uint2 *>(&T.Wt[b][tid >> 7][0])[tid & 127] =
              uint2{wring[d][0], wring[d][1]};
        else
          *reinterpret_cast<u32x4 *>(&T.Wt[b][tid >> 7][tid & 127]) = wring[d];
        if (chunk_fastest) {
          if (++cs == chunks) {
            cs = 0;
            ks = min(ks + 1, kn - 1);
          }
        } else if (++ks == kn) {
          ks = 0;
        }
      };
      auto products = [&](int b) {
        const bf16x8 bq = __builtin_bit_cast(bf16x8, T.S[b][lhi][wave * 32 + l31]);
        bf16x8 aq[2 * OG];
#pragma unroll
        for (int m = 0; m < 2 * OG; m++)
          aq[m] = __builtin_bit_cast(bf16x8, T.Wt[b][lhi][32 * m + l31]);
#pragma unroll
        for (int m = 0; m < 2 * OG; m++)
          acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aq[m], bq, acc[m], 0, 0, 0);
      };
#pragma unroll
      for (int d = 0; d < kDepth; d++) issue_slot(d);
      int u = 0;
      for (; u + kDepth <= units; u += kDepth) {  // whole rounds of the ring, branch-free
#pragma unroll
        for (int d = 0; d < kDepth; d++) {
          stage_slot(d, buf);
          __syncthreads();
          issue_slot(d);
          products(buf);
          buf ^= 1;
        }
      }
#pragma unroll
      for (int d = 0; d < kDepth - 1; d++) {  // the last units, already in flight
        if (u + d < units) {
          stage_slot(d, buf);
          __syncthreads();
          products(buf);
          buf ^= 1;
        }
      }
      continue;
    }
    load_tap(0);
    set_chunk(0);
    issue(k0, 0);
    int kl = 0, c = 0;
    for (int u = 0; u < units; ++u) {
      stage(buf);
      __syncthreads();
      if (chunk_fastest) {
        if (++c == chunks) {
          c = 0;
          ++kl;
        }
        set_chunk(c);
      } else if (++kl == kn) {
        kl = 0;
        ++c;
        set_chunk(c);
      }
      if (u + 1 < units) {  // next unit's taps and gathers in flight during the MFMAs
        load_tap(kl);
        issue(k0 + kl, c);
      }
      // fetch every operand of the chunk first, then issue the MFMAs back to back
      if constexpr (kBf16) {
        const bf16x8 bq = __builtin_bit_cast(bf16x8, T.S[buf][lhi][wave * 32 + l31]);
        bf16x8 aq[2 * OG];
#pragma unroll
        for (int m = 0; m < 2 * OG; m++)
          aq[m] = __builtin_bit_cast(bf16x8, T.Wt[buf][lhi][32 * m + l31]);
#pragma unroll
        for (int m = 0; m < 2 * OG; m++)
          acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aq[m], bq, acc[m], 0, 0, 0);
      } else {
        float bv[kGC / 2], av[2 * OG][kGC / 2];
#pragma unroll
        for (int s = 0; s < kGC / 2; s++) {
          const int kk = 2 * s + lhi;
          bv[s] = T.S[buf][kk][wave * 32 + l31];
#pragma unroll
          for (int m = 0; m < 2 * OG; m++) av[m][s] = T.Wt[buf][kk][32 * m + l31];
        }
#pragma unroll
        for (int s = 0; s < kGC / 2; s++)
#pragma unroll
          for (int m = 0; m < 2 * OG; m++)
            acc[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[m][s], bv[s], acc[m], 0, 0, 0);
      }
      buf ^= 1;
    }
  }

  // epilogue: lane holds pixel (wave*32 + l31) and 2 x 16 output channels
  const int pe = wave * 32 + l31;
  const int ei = tile_y * th + (pe >> tw_shift), ej = (tile_x << tw_shift) + (pe & tw_mask);
  if (ei < OH && ej < OW) {
    TD *yb = y + (int64_t)b * O * N + (int64_t)ei * OW + ej;
    // `addend`: a channel-last fp32 image [B][N][Opad] of contributions accumulated elsewhere
    // (the overflow list of a transposed map, gate[1] entries long), added when there are any
    const float *ab = (addend && gate && gate[1] > 0)
                          ? addend + ((int64_t)b * N + (int64_t)ei * OW + ej) * Opad
                          : nullptr;
#pragma unroll
    for (int m = 0; m < 2 * OG; m++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int o = o0 + 32 * m + (i >> 2) * 8 + lhi * 4 + (i & 3);
        if (o < O) {
          const float start = accumulate ? to_f32(yb[(int64_t)o * N]) : (bias ? to_f32(bias[o]) : 0.f);
          yb[(int64_t)o * N] = from_f32<TD>(acc[m][i] + start + (ab ? ab[o] : 0.f));
        }
      }
  }
}

// ---------------------------------------------------------------------------------
// gather_product for bf16 images, direct form.  With bf16 MFMA the products of a unit (one
// tap x 16 source channels) are short, and matrix and vector instructions of a SIMD all but
// take turns: the general kernel above spends its time on the vector instructions around the
// samples (unpacking, fp32 interpolation, the way through LDS) and on re-reading the weight
// tile once per 32 pixels.  Here
//   * a lane gathers and interpolates exactly the elements its MFMA B operand holds
//     (v_mfma_f32_32x32x16_bf16: lane (l31, lhi) holds channels lhi*8 .. lhi*8+7 of pixel column
//     l31), so samples never touch LDS, and a wave multiplies two 32-pixel blocks by all 64*OG
//     output channels per weight fetch: half the LDS bytes per product;
//   * a tap is NA (pixel, weight) entries; a 32-bit word of an entry (two channels of its
//     pixel) is multiplied by {w, 0} for the even and by {0, w} for the odd channel with
//     v_dot2_f32_bf16: one instruction per channel and entry, nothing to unpack (v_perm_b32,
//     which could bring the same channel of two pixels into one word, runs at half rate).  The
//     weights are rounded to bf16, the precision of the samples they multiply;
//   * gathers are buffer loads (scalar block offset + the lane's 32-bit offset: no address
//     arithmetic in the loop), the loads of kDepth units are in flight, and the LDS reads of a
//     unit are issued a step ahead of their use.
// Only the weights (linear copies of the pre-packed slices) go through LDS, double buffered,
// one barrier per unit.  A workgroup is 4 waves = 256 consecutive pixels of an image (in the
// order of the flattened map, so any image width works) x 64*OG output channels.  The source is
// the copy in blocks of 8 channels per pixel (to_channel_blocks_kernel).  PACKED: the taps come
// from a packed map (a transposed map or a plan's gather part: four (pixel, weight) entries per
// tap); else from sample_map under single-point bilinear / bispherical interpolation.  NA counts
// the leading entries of a tap that are read (2 or 4); the launches of both values are gated
// like those of the general kernel (pair_mask / row_mask).
constexpr int kDgPx = 256;

template <bool PACKED, int NA, int OG>
__global__ __launch_bounds__(kThreads, 2) void gather_product_bf16_direct_kernel(
    const bf16_t *__restrict__ src, const float *__restrict__ map, const float *__restrict__ iw,
    const uint16_t *__restrict__ wb, const bf16_t *__restrict__ bias, bf16_t *__restrict__ y,
    int O, int Opad, int Gpad, int SH, int SW, int N, int OW, int K, int weighted, int wrap,
    int tiles_per_img, const int *__restrict__ gate, int run_if_zero,
    const float *__restrict__ addend, const int *__restrict__ pair_mask, int run_if_leading,
    const int *__restrict__ row_mask, int mask_words) {
  static_assert(NA == 2 || NA == 4, "two or four entries per tap");
  constexpr int NPR = NA / 2;              // entry pairs per tap
  constexpr int TG = NA <= 2 ? 13 : 4;     // taps resolved into LDS at a time
  constexpr int kDepth = NA <= 2 ? 3 : 2;  // units whose loads are in flight
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) unsigned TapOff[TG][kDgPx][NA];
  __shared__ __attribute__((aligned(16))) unsigned TapW[TG][kDgPx][NA];  // bf16 weights as {w, 0}
  __shared__ __attribute__((aligned(16))) uint4 Wt[2][2][kOT * OG];
  if (gate && ((*gate == 0) != (run_if_zero != 0))) return;  // device-side path selection
  const int tid = threadIdx.x;
  const int tile = xcd_contiguous_tile(blockIdx.x, gridDim.x);
  const int b = tile / tiles_per_img;
  const int n0 = (tile - b * tiles_per_img) * kDgPx;
  if (pair_mask) {
    // the two-entry form serves every tile none of whose rows uses a later entry
    bool leading = !later_pairs_in_use(pair_mask, mask_words);
    if (!leading && row_mask) {
      int any = 0;
      for (int r = n0 / OW; r <= min(n0 + kDgPx - 1, N - 1) / OW; r++) any |= row_mask[r];
      leading = any == 0;
    }
    if (leading != (run_if_leading != 0)) return;
  }
  const int o0 = blockIdx.y * (kOT * OG);
  const int64_t plane = (int64_t)SH * SW;
  const unsigned bstride = (unsigned)plane * 16u;  // bytes of a block of 8 channels of an image
  const int chunks = Gpad / kGC;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, lhi = lane >> 5;
  const int px[2] = {wave * 64 + l31, wave * 64 + 32 + l31};  // this lane's pixels of the tile
  // the image's staged copy as a buffer: the lane's offset selects pixel and (through lhi) the
  // upper or lower block of a chunk, the scalar offset the chunk
  const auto img = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(src) + (int64_t)b * Gpad * plane, (short)0,
      (int)((unsigned)(Gpad / 8) * bstride), 0x00020000);
  const unsigned lane_block = (unsigned)lhi * bstride;
  const auto wbuf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(wb), (short)0, (int)((unsigned)K * chunks * 2u * Opad * 16u),
      0x00020000);
  // this thread's 16 bytes of a unit's weights: [kg][output][8 channels]
  constexpr int kPerKg = kOT * OG;
  const int wt = min(tid, 2 * kPerKg - 1);
  const unsigned w_lane = ((unsigned)(wt / kPerKg) * Opad + o0 + wt % kPerKg) * 16u;

  floatx16 acc[2 * OG][2];
#pragma unroll
  for (int m = 0; m < 2 * OG; m++)
#pragma unroll
    for (int q = 0; q < 2; q++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[m][q][i] = 0.f;

  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += TG) {
    const int kn = min(TG, K - k0);
    __syncthreads();  // the previous group's units are done with the tap cache
    {                 // thread tid resolves the group's taps of pixel tid
      const int n = n0 + tid;
      const bool live = n < N;
      const int64_t ng = live ? n : 0;
      for (int kl = 0; kl < kn; kl++) {
        unsigned off[4];
        float wgt[4];
        if constexpr (PACKED) {
          // pre-resolved entries [tap][slot][pixel]: (pixel index of the source as bits, weight)
#pragma unroll
          for (int r = 0; r < NA; r++) {
            const float2 q =
                reinterpret_cast<const float2 *>(map)[((int64_t)(k0 + kl) * 4 + r) * N + ng];
            off[r] = __builtin_bit_cast(unsigned, q.x) * 16u;
            wgt[r] = live ? q.y : 0.f;
          }
        } else {
          const int64_t e = ng * K + k0 + kl;
          PairTap<4> t;
          resolve_pairs<4, 16>(map[e * 2], map[e * 2 + 1], SH, SW, wrap != 0,
                               live ? (weighted ? iw[e] : 1.f) : 0.f, t);
#pragma unroll
          for (int r = 0; r < NA; r++) {
            off[r] = t.off[r];
            wgt[r] = t.wt[r];
          }
        }
#pragma unroll
        for (int r = 0; r < NA; r++) TapOff[kl][tid][r] = off[r];
        // entry r weighs w[r] (rounded to bf16, the precision of the samples themselves), kept
        // as the word {w, 0} that weighs the even channel of a sample word; a lane-side shift
        // makes the {0, w} of the odd one
#pragma unroll
        for (int r = 0; r < NA; r++)
          TapW[kl][tid][r] = __builtin_bit_cast(
              unsigned, __builtin_convertvector(floatx2{wgt[r], 0.f}, bf16x2));
      }
    }
    __syncthreads();

    // units: chunk-major, the tap fastest (a chunk's source rows stay in cache for all taps)
    const int units = chunks * kn;
    u32x4 ring[kDepth][2][NA];
    u32x4 wring[kDepth];
    int ki = 0, ci = 0, ks = 0;
    // `offn`: the offsets of the unit whose loads are issued next; `wnext`: the packed weights
    // of the unit that is interpolated next (both read from LDS a step ahead)
    unsigned offn[2][NA], wnext[2][NA];
    auto fetch_offsets = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < 2; q++)
#pragma unroll
        for (int r = 0; r < NA; r++) offn[q][r] = TapOff[ki][px[q]][r] + lane_block;
    };
    auto fetch_weights = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < 2; q++)
#pragma unroll
        for (int r = 0; r < NA; r++) wnext[q][r] = TapW[ks][px[q]][r];
    };
    auto issue_slot = [&](int d) __attribute__((always_inline)) {
      // (wave-uniform by construction; said so explicitly, or the loads get a loop over lanes)
      const int cc = __builtin_amdgcn_readfirstlane(min(ci, chunks - 1));
      const int chunk_off = (int)((unsigned)cc * 2u * bstride);
      const int w_off = __builtin_amdgcn_readfirstlane(
          (int)((unsigned)((k0 + ki) * chunks + cc) * 2u * (unsigned)Opad * 16u));
#pragma unroll
      for (int q = 0; q < 2; q++)
#pragma unroll
        for (int r = 0; r < NA; r++)
          ring[d][q][r] = __builtin_bit_cast(
              u32x4, __builtin_amdgcn_raw_buffer_load_b128(img, (int)offn[q][r], chunk_off, 0));
      wring[d] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(wbuf, (int)w_lane, w_off, 0));
      if (++ki == kn) {
        ki = 0;
        ++ci;
      }
    };
    bf16x8 bq[2];
    auto stage_slot = [&](int d, int bb) __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < 2; q++) {
        float sv[8];
#pragma unroll
        for (int r = 0; r < NPR; r++) {
          // a word of an entry holds channels 2j (low half) and 2j + 1 of its pixel: against
          // {w, 0} the dot product weighs the even channel, against {0, w} the odd one
          const unsigned w_even[2] = {wnext[q][2 * r], wnext[q][2 * r + 1]};
          const unsigned w_odd[2] = {w_even[0] << 16, w_even[1] << 16};
#pragma unroll
          for (int e = 0; e < 2; e++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
              const unsigned word = ring[d][q][2 * r + e][j];
              if (r == 0 && e == 0) {
                sv[2 * j] = dot_bf16_first(word, w_even[e]);
                sv[2 * j + 1] = dot_bf16_first(word, w_odd[e]);
              } else {
                sv[2 * j] = dot_bf16(word, w_even[e], sv[2 * j]);
                sv[2 * j + 1] = dot_bf16(word, w_odd[e], sv[2 * j + 1]);
              }
            }
        }
        u32x4 pk;
#pragma unroll
        for (int j = 0; j < 4; j++)
          pk[j] = __builtin_bit_cast(
              unsigned, __builtin_convertvector(floatx2{sv[2 * j], sv[2 * j + 1]}, bf16x2));
        bq[q] = __builtin_bit_cast(bf16x8, pk);
      }
      if (tid < 2 * kPerKg)
        *reinterpret_cast<u32x4 *>(&Wt[bb][tid / kPerKg][tid % kPerKg]) = wring[d];
      if (++ks == kn) ks = 0;
    };
    bf16x8 aq[2 * OG];
    auto fetch_operands = [&](int bb) __attribute__((always_inline)) {
#pragma unroll
      for (int m = 0; m < 2 * OG; m++)
        aq[m] = __builtin_bit_cast(bf16x8, Wt[bb][lhi][32 * m + l31]);
    };
    auto products = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int m = 0; m < 2 * OG; m++)
#pragma unroll
        for (int q = 0; q < 2; q++)
          acc[m][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aq[m], bq[q], acc[m][q], 0, 0, 0);
    };
    // (loads are issued unconditionally, past the last unit too, where they read the last
    // chunk again: a load behind a branch would make every later wait a full one)
    fetch_offsets();
#pragma unroll
    for (int d = 0; d < kDepth; d++) {
      issue_slot(d);
      fetch_offsets();
    }
    fetch_weights();
    int u = 0;
    for (; u + kDepth <= units; u += kDepth) {
#pragma unroll
      for (int d = 0; d < kDepth; d++) {
        stage_slot(d, buf);
        __syncthreads();
        fetch_operands(buf);
        fetch_weights();
        issue_slot(d);
        fetch_offsets();
        products();
        buf ^= 1;
      }
    }
#pragma unroll
    for (int d = 0; d < kDepth - 1; d++) {
      if (u + d < units) {
        stage_slot(d, buf);
        __syncthreads();
        fetch_operands(buf);
        fetch_weights();
        products();
        buf ^= 1;
      }
    }
  }

  // epilogue: block (m, q) of the lane holds pixel px[q] and 16 output channels, consecutive
  // ones in consecutive elements.  Neighbouring lanes hold neighbouring pixels: with an even
  // pixel count per plane a pair of lanes swaps one value of every two channels, so that the
  // even lane stores two pixels of the even channel in one 32-bit word and the odd lane two
  // pixels of the odd channel (half the store instructions of 2-byte stores).
  const float *ab_img = (addend && gate && gate[1] > 0) ? addend : nullptr;
  const bool pack2 = (N & 1) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;
  const bool odd = (l31 & 1) != 0;
#pragma unroll
  for (int q = 0; q < 2; q++) {
    const int n = n0 + px[q];
    if (n >= N) continue;
    bf16_t *yb = y + (int64_t)b * O * N + n;
    const float *ab = ab_img ? ab_img + ((int64_t)b * N + n) * Opad : nullptr;
#pragma unroll
    for (int m = 0; m < 2 * OG; m++)
#pragma unroll
      for (int t = 0; t < 8; t++) {
        const int oa = o0 + 32 * m + (t >> 1) * 8 + lhi * 4 + (t & 1) * 2, ob = oa + 1;
        // (channels past O read a valid bias element; they are not stored)
        const float va = acc[m][q][2 * t] + (bias ? to_f32(bias[min(oa, O - 1)]) : 0.f) +
                         (ab ? ab[oa] : 0.f);
        const float vb = acc[m][q][2 * t + 1] + (bias ? to_f32(bias[min(ob, O - 1)]) : 0.f) +
                         (ab ? ab[ob] : 0.f);
        if (pack2) {
          const float send = odd ? va : vb;
          const float recv = __builtin_bit_cast(
              float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, send), 0xB1, 0xf, 0xf,
                                              true));  // quad_perm [1, 0, 3, 2]
          const int o = odd ? ob : oa;
          const unsigned two = __builtin_bit_cast(
              unsigned, __builtin_convertvector(floatx2{odd ? recv : va, odd ? vb : recv}, bf16x2));
          if (o < O)
            *reinterpret_cast<unsigned *>(yb + (int64_t)o * N - (odd ? 1 : 0)) = two;
        } else {
          if (oa < O) yb[(int64_t)oa * N] = from_f32<bf16_t>(va);
          if (ob < O) yb[(int64_t)ob * N] = from_f32<bf16_t>(vb);
        }
      }
  }
}

// ---------------------------------------------------------------------------------
// weight_grad: gW[a,g,k] = sum_{b,n} plain[b,a,n] * sample(gath[b,g], map[n,k])
// (convolution: plain = grad_output, gath = input; transposed: plain = input,
// gath = grad_output).  The reduction dimension is the pixel axis, so a workgroup
// walks a range of pixel tiles and keeps its slice of gW in MFMA accumulators:
// 64 plain channels x 32 gathered channels x up to 9 taps (fp32; bf16 storage: 128 x 16 x 9).
// Per tile the plain tile P[64][128] is staged in LDS once and each wave keeps its 16 rows
// as MFMA A operands in registers; per (tap, 16-channel block) the gathered samples go to
// LDS as S[16][128] (same gather as the forward kernel) and every wave issues 32
// v_mfma_f32_16x16x4_f32 (bf16: 8 v_mfma_f32_16x16x32_bf16).  Each workgroup writes its partial gW to scratch; a
// second kernel sums the partials in a fixed order (deterministic result).
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Plain channels and 16-channel blocks of gathered channels per workgroup.  With bf16 storage
// the gather bounds the kernel, not the MFMAs: a workgroup then takes 128 plain channels (two
// 16-row blocks per wave) against one block of gathered channels, so that a convolution of up
// to 128 output channels gathers every sample once.
template <typename TD>
constexpr int wg_plain_channels() { return sizeof(TD) == 2 ? 128 : 64; }
template <typename TD>
constexpr int wg_gathered_blocks() { return sizeof(TD) == 2 ? 1 : 2; }
constexpr int kWgKT = 9;            // taps per pass (accumulators in registers)
constexpr int kLdPx = kTilePx + 4;  // LDS row stride (floats)

// The consumers of a pair mask only ask whether a pair beyond the first two is in use
// (mask >= 4).  Accesses to the one address are served one at a time (about 12 ns each), so a
// workgroup reports only when it has such a pair and nobody has reported one yet.
__device__ inline void report_pairs_beyond_two(int *mask, unsigned block_mask) {
  if (threadIdx.x == 0 && block_mask >= 4u &&
      (unsigned)__hip_atomic_load(mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < 4u)
    atomicOr(mask, (int)block_mask);
}

// mask[0] >= 4 iff some sample of the map has a nonzero weight in a pair (point * NCORN +
// corner) beyond the first two.  Grid-stride over the samples.
template <int NCORN>
__global__ void map_pair_mask_kernel(const float *__restrict__ map, const float *__restrict__ iw,
                                     int *__restrict__ mask, int np, int weighted, int wrap,
                                     int GH, int GW, int64_t total) {
  const unsigned m = block_pair_mask<NCORN>(map, iw, np, weighted, wrap, GH, GW, total,
                                            (int)blockIdx.x, (int)gridDim.x);
  if (gridDim.x == 1) {  // a launch of one block owns the word: no clearing before it
    if (threadIdx.x == 0) *mask = (int)m;
    return;
  }
  report_pairs_beyond_two(mask, m);
}

// CL: `gath` is a channel-last copy [B][GH*GW][Gpad] of the gathered operand (see the
// gather-product kernel).
// NA: leading (offset, weight) pairs of a tap that are loaded and added.  NA < NP*NCORN is
// valid when the remaining pairs are zero for every sample of the map (bilinear corners of
// integral row coordinates, unused points); map_pair_mask_kernel finds that out on the
// device and `pair_mask` / `run_if_leading` let exactly one of two launched variants run.
template <typename TD, int NCORN, int NP, bool CL, int NA>
__global__ __launch_bounds__(kThreads, NP * NCORN <= 4 ? 3 : 2) void weight_grad_mfma_kernel(
    const TD *__restrict__ plain, const TD *__restrict__ gath,
    const float *__restrict__ map, const float *__restrict__ iw, float *__restrict__ part, int A,
    int G, int GH, int GW, int MH, int MW, int K, int weighted, int wrap, int tiles_x,
    int tiles_per_img, int tw_shift, int total_tiles, int ranges, int cgroups,
    float *__restrict__ plain_sum_part, const int *__restrict__ pair_mask, int run_if_leading,
    const uint4 *__restrict__ tap_table) {
  constexpr int NE = NP * NCORN;  // (offset, weight) pairs per pixel and tap
  static_assert(NA >= 1 && NA <= NE, "NA counts leading pairs");
  // two variants are launched, with NA == 2 (run_if_leading) and NA == NE; the map's mask of
  // pairs in use decides which of them does the work
  if (pair_mask && (((unsigned)*pair_mask < (1u << 2)) != (run_if_leading != 0))) return;
  // The plain tile is only needed until each wave has copied its rows into registers;
  // the same LDS then holds the tile's resolved taps (offsets, then weights).
  // bf16 storage: both tiles hold bf16 (row stride kLdPxB keeps 16-byte row reads of 16
  // different rows on different banks) and feed v_mfma_f32_16x16x32_bf16, whose lanes take
  // 8 consecutive pixels of their row.
  constexpr bool kBf16 = sizeof(TD) == 2;
  constexpr int kLdPxB = kTilePx + 8;
  constexpr int kWgA = wg_plain_channels<TD>(), kWgCB = wg_gathered_blocks<TD>();
  constexpr int MB = kWgA / 64;  // 16-row blocks of plain channels per wave
  constexpr int kPtFloats = kBf16 ? kWgA * kLdPxB / 2 : kWgA * kLdPx;
  constexpr int kTapFloats = 2 * kWgKT * kTilePx * NA;
  constexpr bool kCacheTaps = kTapFloats <= kPtFloats + 1024;
  __shared__ __attribute__((aligned(16))) float PtMem[kCacheTaps && kTapFloats > kPtFloats ? kTapFloats : kPtFloats];
  __shared__ __attribute__((aligned(16))) float SMem[kBf16 ? kGC * kLdPxB : 2 * kGC * kLdPx];
  float(*Pt)[kLdPx] = reinterpret_cast<float(*)[kLdPx]>(PtMem);
  float(*S)[kGC][kLdPx] = reinterpret_cast<float(*)[kGC][kLdPx]>(SMem);
  uint16_t(*PtB)[kLdPxB] = reinterpret_cast<uint16_t(*)[kLdPxB]>(PtMem);
  uint16_t(*SB)[kGC][kLdPxB] = reinterpret_cast<uint16_t(*)[kGC][kLdPxB]>(SMem);
  // (NA pairs per pixel: with two, a lane's offsets are one 8-byte word and the lanes of a
  // wave read consecutive words)
  unsigned(*TapOff)[kTilePx][NA] = reinterpret_cast<unsigned(*)[kTilePx][NA]>(PtMem);
  float(*TapWt)[kTilePx][NA] =
      reinterpret_cast<float(*)[kTilePx][NA]>(PtMem + kWgKT * kTilePx * NA);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l15 = lane & 15, lq = lane >> 4;
  int range, cg;
  if ((ranges & 7) == 0) {  // channel groups of one pixel range share an XCD (and its L2)
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    cg = slot % cgroups;
    range = xcd * (ranges >> 3) + slot / cgroups;
  } else {
    cg = blockIdx.x % cgroups;
    range = blockIdx.x / cgroups;
  }
  const int a0 = blockIdx.y * kWgA;
  const int k_base = blockIdx.z * kWgKT;
  const int ktaps = min(kWgKT, K - k_base);
  const int tpr = (total_tiles + ranges - 1) / ranges;
  const int t_begin = range * tpr, t_end = min(total_tiles, t_begin + tpr);
  const int tw_mask = (1 << tw_shift) - 1, th = kTilePx >> tw_shift;
  const int N = MH * MW;
  const int64_t gplane = (int64_t)GH * GW;
  const int p = tid & (kTilePx - 1);
  const int half = __builtin_amdgcn_readfirstlane(tid >> 7);  // wave-uniform: scalar addressing
  const int g_first = cg * (kWgCB * kGC);
  // 16-byte loads of the plain tile need every row segment 16-byte aligned
  const bool vec_ok = (MW & (16 / (int)sizeof(TD) - 1)) == 0 &&
                      (reinterpret_cast<uintptr_t>(plain) & 15) == 0;

  floatx4 acc[kWgKT][kWgCB][MB];
#pragma unroll
  for (int k = 0; k < kWgKT; k++)
#pragma unroll
    for (int cb = 0; cb < kWgCB; cb++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++) acc[k][cb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};
  // Sum of the plain operand over pixels (the bias gradient of a convolution), taken from
  // the staged tiles by the workgroups of the first channel group and tap pass: thread
  // (row tid/4 of each 64, quarter tid%4) adds 32 pixels of its row per tile.
  const bool sum_plain = plain_sum_part != nullptr && cg == 0 && blockIdx.z == 0;
  float plain_sum[MB];
#pragma unroll
  for (int mb = 0; mb < MB; mb++) plain_sum[mb] = 0.f;

  for (int tile = t_begin; tile < t_end; ++tile) {
    const int b = tile / tiles_per_img;
    const int t_in = tile - b * tiles_per_img;
    const int tile_y = t_in / tiles_x, tile_x = t_in - tile_y * tiles_x;
    const int i0 = tile_y * th, j0 = tile_x << tw_shift;

    __syncthreads();  // everyone is done with the previous tile's LDS contents
    {
      // A row of the plain tile is kLanesPerRow 16-byte pieces; consecutive lanes take
      // consecutive pieces of a row, so the loads coalesce and the LDS stores of a wave
      // fall into consecutive banks.  A piece never straddles two image rows (either
      // tile shape, 4 x 32 or 1 x 128, is made of 32-pixel runs).
      constexpr int kPer = 16 / (int)sizeof(TD);
      constexpr int kLanesPerRow = kTilePx / kPer, kRowsPerPass = kThreads / kLanesPerRow;
      constexpr int kPasses = kWgA / kRowsPerPass;
      const int px0 = (tid % kLanesPerRow) * kPer;
      const int si = i0 + (px0 >> tw_shift), sj = j0 + (px0 & tw_mask);
      uint4 raw[kPasses];
#pragma unroll
      for (int r = 0; r < kPasses; r++) {
        const int a = tid / kLanesPerRow + r * kRowsPerPass;
        const bool row_ok = (a0 + a) < A && si < MH;
        const TD *prow = plain + ((int64_t)b * A + min(a0 + a, A - 1)) * N +
                         (int64_t)min(si, MH - 1) * MW;
        if (vec_ok && row_ok && sj + kPer <= MW) {
          raw[r] = *reinterpret_cast<const uint4 *>(prow + sj);
        } else {
          TD e[kPer];
#pragma unroll
          for (int q = 0; q < kPer; q++)
            e[q] = (row_ok && sj + q < MW) ? prow[min(sj + q, MW - 1)] : TD{};
          raw[r] = *reinterpret_cast<const uint4 *>(e);
        }
      }
#pragma unroll
      for (int r = 0; r < kPasses; r++) {
        const int a = tid / kLanesPerRow + r * kRowsPerPass;
        if constexpr (kBf16)
          *reinterpret_cast<uint4 *>(&PtB[a][px0]) = raw[r];
        else
          *reinterpret_cast<uint4 *>(&Pt[a][px0]) = raw[r];
      }
    }
    __syncthreads();
    float areg[kBf16 ? 1 : 32];
    bf16x8 aregb[MB][kBf16 ? 4 : 1];
    if constexpr (kBf16) {
#pragma unroll
      for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int s = 0; s < 4; s++)
          aregb[mb][s] = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4 *>(
                          &PtB[(wave * MB + mb) * 16 + l15][32 * s + 8 * lq]));
    } else {
#pragma unroll
      for (int s4 = 0; s4 < 8; s4++) {
        const float4 t =
            *reinterpret_cast<const float4 *>(&Pt[wave * 16 + l15][16 * s4 + 4 * lq]);
        areg[4 * s4 + 0] = t.x;
        areg[4 * s4 + 1] = t.y;
        areg[4 * s4 + 2] = t.z;
        areg[4 * s4 + 3] = t.w;
      }
    }

    if (sum_plain) {
      float t = 0.f;
      if constexpr (kBf16) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
          const uint4 *row =
              reinterpret_cast<const uint4 *>(&PtB[64 * mb + (tid >> 2)][(tid & 3) * 32]);
          t = 0.f;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const uint4 q = row[r];
            const unsigned w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; j++)
              t += __builtin_bit_cast(float, w4[j] << 16) +
                   __builtin_bit_cast(float, w4[j] & 0xffff0000u);
          }
          if (mb + 1 < MB) plain_sum[mb] += t;
        }
      } else {
        const float4 *row = reinterpret_cast<const float4 *>(&Pt[tid >> 2][(tid & 3) * 32]);
#pragma unroll
        for (int r = 0; r < 8; r++) {
          const float4 q = row[r];
          t += (q.x + q.y) + (q.z + q.w);
        }
      }
      plain_sum[MB - 1] += t;
    }

    const int gi = i0 + (p >> tw_shift), gj = j0 + (p & tw_mask);
    const bool live = gi < MH && gj < MW;
    const int64_t n_g = live ? (int64_t)gi * MW + gj : 0;
    const int Gpad = (G + kGC - 1) / kGC * kGC;
    const TD *gath_b = gath + (int64_t)b * (CL ? Gpad : G) * gplane;

    unsigned off[NE];
    float wt[NE];
    float v[8][NE];
    auto resolve_tap = [&](int k, unsigned *o, float *w_) {  // tap k of this thread's pixel
#pragma unroll
      for (int sp = 0; sp < NP; sp++) {
        const int64_t e = (n_g * K + k) * NP + sp;
        PairTap<NCORN> t;
        resolve_pairs<NCORN, sizeof(TD)>(map[e * 2], map[e * 2 + 1], GH, GW, wrap != 0,
                                         live ? (weighted ? iw[e] : 1.f) : 0.f, t);
#pragma unroll
        for (int i = 0; i < NCORN; i++) {
          o[sp * NCORN + i] = CL ? t.off[i] * (unsigned)Gpad : t.off[i];
          w_[sp * NCORN + i] = t.wt[i];
        }
      }
    };
    auto load_tap = [&](int k) {  // k: tap within this pass
      if (kCacheTaps) {
#pragma unroll
        for (int i = 0; i < NA; i++) {
          off[i] = TapOff[k][p][i];
          wt[i] = TapWt[k][p][i];
        }
      } else {
        resolve_tap(k_base + k, off, wt);
      }
    };
    auto issue = [&](int cb) {
      const int g0 = g_first + cb * kGC + half * 8;
      if constexpr (CL) {
        // 8 contiguous channels of the pixel row; a workgroup whose channels lie past the
        // padded count reads the last valid group (its products are not stored)
        const char *base = reinterpret_cast<const char *>(gath_b + min(g0, Gpad - 8));
#pragma unroll
        for (int i = 0; i < NA; i++) {
          const char *row = base + off[i];
          if constexpr (kBf16) {
            const uint4 q = *reinterpret_cast<const uint4 *>(row);
            const unsigned w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
              v[2 * j][i] = __builtin_bit_cast(float, w4[j] << 16);
              v[2 * j + 1][i] = __builtin_bit_cast(float, w4[j] & 0xffff0000u);
            }
          } else {
            const float4 q0 = reinterpret_cast<const float4 *>(row)[0];
            const float4 q1 = reinterpret_cast<const float4 *>(row)[1];
            v[0][i] = q0.x; v[1][i] = q0.y; v[2][i] = q0.z; v[3][i] = q0.w;
            v[4][i] = q1.x; v[5][i] = q1.y; v[6][i] = q1.z; v[7][i] = q1.w;
          }
        }
      } else {
#pragma unroll
        for (int ch = 0; ch < 8; ch++) {
          const TD *pl = gath_b + (int64_t)min(g0 + ch, G - 1) * gplane;
#pragma unroll
          for (int i = 0; i < NA; i++) v[ch][i] = load_at(pl, off[i]);
        }
      }
    };
    auto stage = [&](int buf) {
      float sv[8];
#pragma unroll
      for (int ch = 0; ch < 8; ch++) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NA; i++) s = __builtin_fmaf(wt[i], v[ch][i], s);
        sv[ch] = s;
      }
      if constexpr (kBf16) {
#pragma unroll
        for (int c2 = 0; c2 < 4; c2++) {  // hardware round-to-nearest-even, two values at a time
          const unsigned pk = __builtin_bit_cast(
              unsigned, __builtin_convertvector(floatx2{sv[2 * c2], sv[2 * c2 + 1]}, bf16x2));
          SB[buf][half * 8 + 2 * c2][p] = (uint16_t)(pk & 0xffffu);
          SB[buf][half * 8 + 2 * c2 + 1][p] = (uint16_t)(pk >> 16);
        }
      } else {
#pragma unroll
        for (int ch = 0; ch < 8; ch++) S[buf][half * 8 + ch][p] = sv[ch];
      }
    };

    // (two-pair taps of an image under fp32: resolved before the launch into a table in tile
    // order, resolve_tap_table_kernel<2, 4, false>, and only copied into the tap cache)
    constexpr bool kTable = sizeof(TD) == 4 && !CL && NA == 2 && NE == 4 && kCacheTaps;
    if (kCacheTaps) {
      // every wave has its A operands in registers: reuse the plain tile's LDS for the
      // resolved taps of this tile (thread (p, half) takes every other tap of pixel p)
      __syncthreads();
      bool from_table = false;
      if constexpr (kTable) {
        if (tap_table) {
          // (fetched only here: held across the plain tile's copy, the entries spill)
          from_table = true;
          const uint4 *te = tap_table + ((int64_t)t_in * K + k_base) * kTilePx + p;
          constexpr int kTapsPerThread = (kWgKT + 1) / 2;
          uint4 tap_entry[kTapsPerThread];
#pragma unroll
          for (int t = 0; t < kTapsPerThread; t++)
            tap_entry[t] = te[(int64_t)min(half + 2 * t, ktaps - 1) * kTilePx];
#pragma unroll
          for (int t = 0; t < kTapsPerThread; t++) {
            const int k = half + 2 * t;
            if (k < ktaps) {
              *reinterpret_cast<uint2 *>(&TapOff[k][p][0]) =
                  make_uint2(tap_entry[t].x, tap_entry[t].y);
              *reinterpret_cast<uint2 *>(&TapWt[k][p][0]) =
                  make_uint2(tap_entry[t].z, tap_entry[t].w);
            }
          }
        }
      }
      if (!from_table)
        for (int k = half; k < ktaps; k += 2) {
          unsigned o[NE];
          float w_[NE];
          resolve_tap(k_base + k, o, w_);
#pragma unroll
          for (int i = 0; i < NA; i++) {
            TapOff[k][p][i] = o[i];
            TapWt[k][p][i] = w_[i];
          }
        }
      __syncthreads();
    }

    // Units run channel-block-major with the tap fastest: the rows a 16-channel block
    // touches are reused by all taps while they are still in cache.
    load_tap(0);
    issue(0);
    int buf = 0;
#pragma unroll
    for (int cb = 0; cb < kWgCB; cb++) {
#pragma unroll
      for (int k = 0; k < kWgKT; k++) {
        if (k < ktaps) {
          buf ^= 1;
          stage(buf);
          __syncthreads();
          if (k + 1 < ktaps) {
            load_tap(k + 1);
            issue(cb);
          } else if (cb + 1 < kWgCB) {
            load_tap(0);
            issue(cb + 1);
          }
          // The products of a unit issue back to back: at the default priority the other
          // waves of the SIMD slip their vector work in between and the matrix pipe idles.
          if constexpr (!kBf16) __builtin_amdgcn_s_setprio(1);
          if constexpr (kBf16) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
              const bf16x8 bq = __builtin_bit_cast(
                  bf16x8, *reinterpret_cast<const uint4 *>(&SB[buf][l15][32 * s + 8 * lq]));
#pragma unroll
              for (int mb = 0; mb < MB; mb++)
                acc[k][cb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aregb[mb][s], bq,
                                                                         acc[k][cb][mb], 0, 0, 0);
            }
          } else {
#pragma unroll
            for (int s4 = 0; s4 < 8; s4++) {
              const float4 bq = *reinterpret_cast<const float4 *>(&S[buf][l15][16 * s4 + 4 * lq]);
              acc[k][cb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[4 * s4 + 0], bq.x, acc[k][cb][0], 0, 0, 0);
              acc[k][cb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[4 * s4 + 1], bq.y, acc[k][cb][0], 0, 0, 0);
              acc[k][cb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[4 * s4 + 2], bq.z, acc[k][cb][0], 0, 0, 0);
              acc[k][cb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[4 * s4 + 3], bq.w, acc[k][cb][0], 0, 0, 0);
            }
          }
          if constexpr (!kBf16) __builtin_amdgcn_s_setprio(0);
        }
      }
    }
  }

  if (sum_plain) {  // the four quarters of a row sit in neighbouring lanes
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
      float t = plain_sum[mb];
      t += __shfl_xor(t, 1);
      t += __shfl_xor(t, 2);
      const int a = a0 + 64 * mb + (tid >> 2);
      if ((tid & 3) == 0 && a < A) plain_sum_part[(int64_t)range * A + a] = t;
    }
  }
  // partial gW of this workgroup, stored [tap][gathered channel][plain channel] (rows padded to
  // a multiple of four): the lane holds gathered channel l15 of each block and four
  // consecutive plain channels a0 + 16*(wave*MB + mb) + 4*lq + i, one 16-byte store
  const int A4 = (A + 3) & ~3;
  float *pr = part + (int64_t)range * A4 * G * K;
#pragma unroll
  for (int k = 0; k < kWgKT; k++) {
    if (k < ktaps) {
#pragma unroll
      for (int cb = 0; cb < kWgCB; cb++) {
        const int g = g_first + cb * kGC + l15;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
          const int a = a0 + (wave * MB + mb) * 16 + lq * 4;
          if (a < A && g < G)
            *reinterpret_cast<floatx4 *>(&pr[((int64_t)(k_base + k) * G + g) * A4 + a]) =
                acc[k][cb][mb];
        }
      }
    }
  }
}

// Sums per-range partials, two independent jobs in one launch (the second may be empty):
//   out[a][g][k] = sum over ranges of part[r][k][g][a]   (rows of A4 >= A entries), and
//   out2[e]      = sum over ranges of part2[r][e].
// 64 x 4 threads: four quarters of the ranges are summed side by side (eight loads in flight
// each) and combined in a fixed order, so the result does not depend on scheduling.
template <typename TD>
__global__ __launch_bounds__(256) void reduce_partials_kernel(
    const float *__restrict__ part, TD *__restrict__ out, int A, int A4, int G, int K,
    const float *__restrict__ part2, TD *__restrict__ out2, int64_t n2, int ranges) {
  __shared__ float quarter[4][64];
  int64_t n = (int64_t)K * G * A4;
  const int blocks1 = (int)((n + 63) / 64);
  int64_t e = (int64_t)blockIdx.x * 64 + threadIdx.x;
  const bool second = (int)blockIdx.x >= blocks1;
  if (second) {
    e -= (int64_t)blocks1 * 64;
    part = part2;
    out = out2;
    n = n2;
  }
  const int per = (ranges + 3) / 4;
  const int r0 = min((int)threadIdx.y * per, ranges), r1 = min(r0 + per, ranges);
  float s = 0.f;
  if (e < n) {
    int r = r0;
    for (; r + 8 <= r1; r += 8) {
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = part[(int64_t)(r + u) * n + e];
#pragma unroll
      for (int u = 0; u < 8; u++) s += t[u];
    }
    for (; r < r1; r++) s += part[(int64_t)r * n + e];
  }
  quarter[threadIdx.y][threadIdx.x] = s;
  __syncthreads();
  if (threadIdx.y == 0 && e < n) {
    int64_t o = e;
    if (!second) {
      const int a = (int)(e % A4);
      const int64_t kg = e / A4;  // k * G + g
      const int g = (int)(kg % G), k = (int)(kg / G);
      if (a >= A) return;
      o = ((int64_t)a * G + g) * K + k;
    }
    out[o] = from_f32<TD>(((quarter[0][threadIdx.x] + quarter[1][threadIdx.x]) +
                           quarter[2][threadIdx.x]) + quarter[3][threadIdx.x]);
  }
}

// ---------------------------------------------------------------------------------
// Weight gradient, bf16 storage, unweighted bilinear taps, gathered operand in blocks of 8
// channels per pixel ([B][Gpad/8][GH*GW][8], to_channel_blocks_kernel).  NA == 2: maps whose
// two lower corners weigh nothing anywhere (integral row coordinates); NA == 4: all others (the
// pair mask of the map lets one of the two launches run).  With bf16 MFMA the products are short
// and the kernel lives or dies by its gather, so this form is built around it:
//   * a thread gathers two neighbouring pixels x 8 channels of a unit (one tap, 32 gathered
//     channels): four 16-byte loads instead of 32 two-byte ones (the texture path resolves
//     four lanes per clock whatever the width), and a channel's two pixels leave as one
//     32-bit LDS store, consecutive lanes to consecutive banks;
//   * NA == 2: the loads of kRgDepth units are in flight, across tile boundaries: the taps of
//     the next tile go into the other half of a double-buffered tap cache and the next tile's
//     plain operand is fetched into a second set of registers while this tile's units are
//     multiplied, so that in the steady state no wave waits for memory at a tile's start.
//     NA == 4 has twice the loads per unit and the same registers: one unit in flight (the
//     next unit's loads are issued before this unit's products), a single tap cache, the first
//     unit of a tile waited for;
//   * every load and store is unconditional (past the range's last tile the last one is
//     fetched again, padded taps weigh zero), so the compiler's waits count exactly;
//   * five taps per pass keep the accumulators at 80 registers, which leaves room for the
//     rings at two workgroups per CU;
//   * what every workgroup of a pixel range would do again is done once, before the launch:
//     the taps are resolved into a table in tile order (resolve_tap_table_kernel) and only
//     copied into the tap cache here, and the plain operand is cut into the MFMA fragments of
//     each tile (to_plain_fragments_kernel), which a wave loads as contiguous kilobytes
//     straight into its operand registers: no LDS tile, no barrier at a tile's start.
// Partial sums leave in the layout of weight_grad_mfma_kernel.

// The taps of a bilinear map resolved once for a weight-gradient kernel, in the order its
// workgroups read them: table[tile of an image][tap][pixel of the tile][NA words of byte
// offsets, then NA words of weights].  ESZ: bytes between neighbouring pixels of the gathered
// operand (16 in a channel block, the element size in a plane); WBF: weights as bf16 in the low
// half of the word (what weight_grad_bf16_ring_kernel multiplies by), else as fp32.  Every
// workgroup of a pixel range (channel groups x tap passes) would otherwise resolve the same
// taps from the map again, about sixty instructions per tap, which is as much as its products
// need.  Pixels outside the image weigh zero.  One workgroup per tile: its threads walk the
// taps of their pixel two apart, so the tile's piece of the map stays in cache.
template <int NA, int ESZ, bool WBF>
__global__ __launch_bounds__(256) void resolve_tap_table_kernel(
    const float *__restrict__ map, unsigned *__restrict__ table, int GH, int GW, int MH, int MW,
    int K, int wrap, int tiles_x, int tw_shift, const int *__restrict__ pair_mask) {
  if (pair_mask && (((unsigned)*pair_mask < (1u << 2)) != (NA == 2))) return;
  const int tile = blockIdx.x, p = threadIdx.x & (kTilePx - 1);
  const int tile_y = tile / tiles_x, tile_x = tile - tile_y * tiles_x;
  const int gi = tile_y * (kTilePx >> tw_shift) + (p >> tw_shift);
  const int gj = (tile_x << tw_shift) + (p & ((1 << tw_shift) - 1));
  const bool live = gi < MH && gj < MW;
  const int64_t n_g = (int64_t)min(gi, MH - 1) * MW + min(gj, MW - 1);
  const float2 *entry = reinterpret_cast<const float2 *>(map) + n_g * K;
  uint4 *out = reinterpret_cast<uint4 *>(table) + ((int64_t)tile * K * kTilePx + p) * (NA / 2);
  // (a weight as bf16 in the low half of a word, the high half zero: the form
  // v_dot2_f32_bf16 multiplies a word of two channels by to get the even one)
  auto wbits = [](float w) {
    return WBF ? __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{w, 0.f}, bf16x2))
               : __builtin_bit_cast(unsigned, w);
  };
  for (int k = threadIdx.x >> 7; k < K; k += 2) {
    const float2 xy = entry[k];
    PairTap<4> t;
    resolve_pairs<4, ESZ>(xy.x, xy.y, GH, GW, wrap != 0, live ? 1.f : 0.f, t);
    uint4 *e = out + (int64_t)k * kTilePx * (NA / 2);
    if constexpr (NA == 2) {
      e[0] = make_uint4(t.off[0], t.off[1], wbits(t.wt[0]), wbits(t.wt[1]));
    } else {
      e[0] = make_uint4(t.off[0], t.off[1], t.off[2], t.off[3]);
      e[1] = make_uint4(wbits(t.wt[0]), wbits(t.wt[1]), wbits(t.wt[2]), wbits(t.wt[3]));
    }
  }
}

constexpr int kRgKT = 5;      // taps per pass
constexpr int kRgG = 32;      // gathered channels per workgroup
constexpr int kRgA = 128;     // plain channels per workgroup
constexpr int kRgDepth = 2;   // units whose gathers are in flight
constexpr int kRgLd = kTilePx + 8;  // bf16 elements per LDS row

inline int ring_weight_grad_ranges(int64_t total_tiles, int64_t A, int64_t G, int64_t K) {
  const int64_t per_range = ((G + kRgG - 1) / kRgG) * ((A + kRgA - 1) / kRgA) *
                            ((K + kRgKT - 1) / kRgKT);
  // about twenty workgroups per CU, two of them resident at a time: they drift apart, and
  // short ones even out the end of the launch (config 5: 27.8 / 26.3 / 25.6 / 25.6 ms per
  // backward call with 1024 / 2560 / 5120 / 10240 workgroups)
  int64_t r = std::max<int64_t>(8, (5120 / per_range) / 8 * 8);
  r = std::min<int64_t>(r, std::max<int64_t>(total_tiles / 8 * 8, 8));
  return (int)r;
}

template <int NA>
__global__ __launch_bounds__(kThreads, 2) void weight_grad_bf16_ring_kernel(
    const bf16_t *__restrict__ plain, const bf16_t *__restrict__ gath,
    const unsigned *__restrict__ table, float *__restrict__ part, int A, int G, int Gpad, int GH,
    int GW, int K, int tiles_per_img, int total_tiles, int ranges, int cgroups, int passes,
    float *__restrict__ plain_sum_part, const int *__restrict__ pair_mask) {
  // NA == 2 runs while no tap of the map uses a pair beyond its first two, NA == 4 otherwise
  if (pair_mask && (((unsigned)*pair_mask < (1u << 2)) != (NA == 2))) return;
  static_assert(NA == 2 || NA == 4, "two or four pairs per tap");
  constexpr bool kCross = NA == 2;               // gathers in flight across tile boundaries
  constexpr int kDepth = kCross ? kRgDepth : 1;  // units in flight
  constexpr int kTapBufs = kCross ? 2 : 1;
  constexpr int MB = kRgA / 64, NB = kRgG / 16;
  __shared__ __attribute__((aligned(16))) uint16_t SB[2][kRgG][kRgLd];
  __shared__ __attribute__((aligned(16))) unsigned TapOff[kTapBufs][kRgKT][kTilePx][NA];
  __shared__ __attribute__((aligned(16))) float TapWt[kTapBufs][kRgKT][kTilePx][NA];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l15 = lane & 15, lq = lane >> 4;
  // the workgroups of one pixel range (channel groups x tap passes) share an XCD and its L2
  const int combos = cgroups * passes;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int combo = slot % combos;
  const int range = xcd * (ranges >> 3) + slot / combos;
  const int cg = combo % cgroups, pass = combo / cgroups;
  const int a0 = blockIdx.y * kRgA;
  const int k_base = pass * kRgKT;
  const int tpr = (total_tiles + ranges - 1) / ranges;
  const int t_begin = range * tpr, t_end = min(total_tiles, t_begin + tpr);
  const int64_t gplane = (int64_t)GH * GW;
  const int g_first = cg * kRgG;

  // roles.  Tap cache: pixel p, taps half, half + 2, ...  Gather: pixel pair pp, the
  // wave's 8 channels.  Plain operand: the wave's own MFMA fragments, straight from memory.
  const int p = tid & (kTilePx - 1), half = tid >> 7;
  const int pp = lane;
  const int64_t group = min(g_first / 8 + wave, Gpad / 8 - 1);  // (past Gpad: not stored)
  constexpr int kTapsPerThread = (kRgKT + 1) / 2;
  static_assert(MB == 2, "a wave's rows are one slab of to_plain_fragments_kernel");
  const int slabs = (A + 31) / 32;

  floatx4 acc[kRgKT][NB][MB];
#pragma unroll
  for (int k = 0; k < kRgKT; k++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++) acc[k][nb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bool sum_plain = plain_sum_part != nullptr && combo == 0;
  float plain_sum[MB];
#pragma unroll
  for (int mb = 0; mb < MB; mb++) plain_sum[mb] = 0.f;

  // plain operand of this tile and of the next, by the tile's parity in the range
  bf16x8 aregb[2][MB][4];
  uint4 tapreg[kTapsPerThread][NA / 2];
  uint4 q[kDepth][2 * NA];  // [unit in flight][pixel of the pair * NA + pair of the tap]

  // (tiles past the range's end, which pad it to a whole number of ring periods, are fetched
  // as zeros and weigh zero; their addresses are those of the last tile)
  // (`plain` is the copy to_plain_fragments_kernel made: the wave's slab of a tile is 8 KB,
  // fragment (mb, s4) a kilobyte of it, a lane's piece 16 bytes; a slab past the last channel
  // does not exist in the copy and a tile past the range's end is not to be read: both get a
  // buffer of no bytes and read as zeros)
  const int slab = blockIdx.y * (kRgA / 32) + wave;
  auto fetch_plain = [&](int tile, const int SET) __attribute__((always_inline)) {
    const bool live = tile < t_end && slab < slabs;
    const auto rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t *>(plain + ((int64_t)min(tile, t_end - 1) * slabs + min(slab, slabs - 1)) * 4096),
        (short)0, live ? 8192 : 0, 0x00020000);
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++)
        aregb[SET][mb][s4] = __builtin_bit_cast(
            bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16, (mb * 4 + s4) * 1024, 0));
  };
  // Entries of `tile` from the table resolve_tap_table_kernel made, into registers: the taps
  // of this pass as a buffer, so that taps past the map's last one and tiles past the range's
  // end read as zeros (offset 0, weight 0).
  auto fetch_taps = [&](int tile) __attribute__((always_inline)) {
    const int taps = tile < t_end ? min(kRgKT, K - k_base) : 0;
    const int t_in = min(tile, t_end - 1) % tiles_per_img;
    const auto rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned *>(table + ((int64_t)t_in * K + k_base) * kTilePx * 2 * NA),
        (short)0, taps * kTilePx * 8 * NA, 0x00020000);
#pragma unroll
    for (int t = 0; t < kTapsPerThread; t++)
#pragma unroll
      for (int h = 0; h < NA / 2; h++)
        tapreg[t][h] = __builtin_bit_cast(
            uint4, __builtin_amdgcn_raw_buffer_load_b128(
                       rsrc, ((half + 2 * t) * kTilePx + p) * 8 * NA + 16 * h, 0, 0));
  };
  // what fetch_taps brought, into half `par` of the tap cache
  auto store_taps = [&](int par) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kTapsPerThread; t++) {
      const int k = half + 2 * t;
      if (k < kRgKT) {
        if constexpr (NA == 2) {
          const uint4 e = tapreg[t][0];
          *reinterpret_cast<uint2 *>(&TapOff[par][k][p][0]) = make_uint2(e.x, e.y);
          *reinterpret_cast<uint2 *>(&TapWt[par][k][p][0]) = make_uint2(e.z, e.w);
        } else {
          *reinterpret_cast<uint4 *>(&TapOff[par][k][p][0]) = tapreg[t][0];
          *reinterpret_cast<uint4 *>(&TapWt[par][k][p][0]) = tapreg[t][1];
        }
      }
    }
  };
  // (the wave's block of 8 channels of an image as a buffer; tap offsets are bytes inside it)
  auto gather_base = [&](int tile) __attribute__((always_inline)) {
    const int b = min(tile, t_end - 1) / tiles_per_img;
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(reinterpret_cast<const char *>(gath) +
                           (((int64_t)b * (Gpad / 8) + group) * gplane) * 16),
        (short)0, (int)((unsigned)gplane * 16u), 0x00020000);
  };
  // (SLOT is a constant once the unit loops are unrolled: the ring stays in registers)
  auto issue = [&](__amdgpu_buffer_rsrc_t base, int par, int k, const int SLOT)
                   __attribute__((always_inline)) {
    // (the 2 * NA offsets of the pixel pair are consecutive words)
    const uint4 *op = reinterpret_cast<const uint4 *>(&TapOff[par][k][2 * pp][0]);
#pragma unroll
    for (int h = 0; h < NA / 2; h++) {
      const uint4 o = op[h];
      const unsigned ov[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
      for (int i = 0; i < 4; i++)
        q[SLOT][4 * h + i] = __builtin_bit_cast(
            uint4, __builtin_amdgcn_raw_buffer_load_b128(base, (int)ov[i], 0, 0));
    }
  };
  auto stage = [&](int par, int k, const int SLOT, int buf) __attribute__((always_inline)) {
    // weights of the pixel pair: NA for the first pixel, then NA for the second
    float wv[2 * NA];
    {
      const float4 *wp4 = reinterpret_cast<const float4 *>(&TapWt[par][k][2 * pp][0]);
#pragma unroll
      for (int h = 0; h < NA / 2; h++) {
        const float4 t = wp4[h];
        wv[4 * h] = t.x; wv[4 * h + 1] = t.y; wv[4 * h + 2] = t.z; wv[4 * h + 3] = t.w;
      }
    }
    // a word of a gathered record holds channels 2j (low half) and 2j + 1: against {w, 0} the
    // two-element dot product weighs the even channel, against {0, w} the odd one (one
    // instruction per sample and pair, nothing to unpack; the weights are bf16 like the samples)
    unsigned w_even[2 * NA], w_odd[2 * NA];
#pragma unroll
    for (int i = 0; i < 2 * NA; i++) {
      w_even[i] = __builtin_bit_cast(unsigned, wv[i]);
      w_odd[i] = w_even[i] << 16;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {  // channels 2j and 2j + 1 of the wave's eight
      float e[2], o[2];  // [pixel of the pair]
#pragma unroll
      for (int px = 0; px < 2; px++)
#pragma unroll
        for (int i = 0; i < NA; i++) {  // in the order of the pairs, like every other kernel
          const uint4 t = q[SLOT][px * NA + i];
          const unsigned word = j == 0 ? t.x : j == 1 ? t.y : j == 2 ? t.z : t.w;
          if (i == 0) {
            e[px] = dot_bf16_first(word, w_even[px * NA]);
            o[px] = dot_bf16_first(word, w_odd[px * NA]);
          } else {
            e[px] = dot_bf16(word, w_even[px * NA + i], e[px]);
            o[px] = dot_bf16(word, w_odd[px * NA + i], o[px]);
          }
        }
      // (hardware round-to-nearest-even, the two pixels of a channel in one word)
      *reinterpret_cast<unsigned *>(&SB[buf][wave * 8 + 2 * j][2 * pp]) =
          __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{e[0], e[1]}, bf16x2));
      *reinterpret_cast<unsigned *>(&SB[buf][wave * 8 + 2 * j + 1][2 * pp]) =
          __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{o[0], o[1]}, bf16x2));
    }
  };

  int buf = 0;
  // One tile.  The ring's period is kRgDepth units and a tile has kRgKT of them, so the slot
  // of a unit depends on the tile's place (PHASE) among kRgDepth consecutive ones: unit k of
  // the tile sits in slot (PHASE * kRgKT + k) % kRgDepth, and the unit issued in its place,
  // kRgDepth units further on, takes the same slot.
  auto run_tile = [&](auto phase_tag, int tile) __attribute__((always_inline)) {
    constexpr int PHASE = decltype(phase_tag)::value;
    // (kCross: `mxy` holds the coordinates of the next tile, whose taps go to the other half
    // of the cache; else those of this tile, resolved now)
    constexpr int SET = PHASE & 1;
    const int par = kCross ? (tile - t_begin) & 1 : 0;
    if constexpr (kCross) {
      // (`tapreg` holds the next tile's taps; the half of the tap cache written here was last
      // read before the previous tile's last barrier, and is first read after this tile's
      // next one)
      store_taps(par ^ 1);
    } else {
      __syncthreads();  // the tap cache is free
      store_taps(0);  // (`tapreg` holds this tile's taps)
      __syncthreads();
    }
    if (sum_plain) {  // the lane adds the 32 pixels it holds of each of its rows
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
        float t = 0.f;
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) {
          const uint4 v = __builtin_bit_cast(uint4, aregb[SET][mb][s4]);
          const unsigned w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int j = 0; j < 4; j++)
            t += __builtin_bit_cast(float, w4[j] << 16) +
                 __builtin_bit_cast(float, w4[j] & 0xffff0000u);
        }
        plain_sum[mb] += t;
      }
    }
    const auto base = gather_base(tile), base_next = gather_base(tile + 1);
    if constexpr (!kCross) issue(base, 0, 0, 0);  // (before the prefetches: it is waited for first)
    fetch_plain(tile + 1, SET ^ 1);
    fetch_taps(kCross ? tile + 2 : tile + 1);
#pragma unroll
    for (int k = 0; k < kRgKT; k++) {
      const int slot_k = (PHASE * kRgKT + k) % kDepth;
      buf ^= 1;
      stage(par, k, slot_k, buf);
      __syncthreads();
      if (k + kDepth < kRgKT)
        issue(base, par, k + kDepth, slot_k);
      else if constexpr (kCross)
        issue(base_next, par ^ 1, k + kDepth - kRgKT, slot_k);
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
          const bf16x8 bq = __builtin_bit_cast(
              bf16x8,
              *reinterpret_cast<const uint4 *>(&SB[buf][nb * 16 + l15][32 * s4 + 8 * lq]));
#pragma unroll
          for (int mb = 0; mb < MB; mb++)
            acc[k][nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aregb[SET][mb][s4], bq,
                                                                     acc[k][nb][mb], 0, 0, 0);
        }
    }
  };

  // prologue: taps of the first tile, its plain operand, coordinates of the second, and the
  // gathers of the first kRgDepth units (a range without tiles stores its zeros)
  static_assert(kRgDepth == 2, "run_tile is instantiated per phase below");
  if (t_begin < t_end) {
    fetch_taps(t_begin);
    if constexpr (kCross) {
      store_taps(0);
      fetch_plain(t_begin, 0);
      fetch_taps(t_begin + 1);
      __syncthreads();
      const auto base0 = gather_base(t_begin);
#pragma unroll
      for (int u = 0; u < kDepth; u++) issue(base0, 0, u, u);
      for (int tile = t_begin; tile < t_end; tile += kDepth) {
        run_tile(std::integral_constant<int, 0>(), tile);
        run_tile(std::integral_constant<int, 1>(), tile + 1);
      }
    } else {
      // (two tiles per turn for the two sets of plain operands; a tile past the end weighs zero)
      fetch_plain(t_begin, 0);
      for (int tile = t_begin; tile < t_end; tile += 2) {
        run_tile(std::integral_constant<int, 0>(), tile);
        run_tile(std::integral_constant<int, 1>(), tile + 1);
      }
    }
  }

  if (sum_plain) {  // the four quarters of a row sit 16 lanes apart
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
      float t = plain_sum[mb];
      t += __shfl_xor(t, 16);
      t += __shfl_xor(t, 32);
      const int a = a0 + (wave * MB + mb) * 16 + l15;
      if (lq == 0 && a < A) plain_sum_part[(int64_t)range * A + a] = t;
    }
  }
  const int A4 = (A + 3) & ~3;
  float *pr = part + (int64_t)range * A4 * G * K;
#pragma unroll
  for (int k = 0; k < kRgKT; k++) {
    if (k_base + k < K) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const int g = g_first + nb * 16 + l15;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
          const int a = a0 + (wave * MB + mb) * 16 + lq * 4;
          if (a < A && g < G)
            *reinterpret_cast<floatx4 *>(&pr[((int64_t)(k_base + k) * G + g) * A4 + a]) =
                acc[k][nb][mb];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// product_scatter: dst[b,d] += splat(sum_s W[s,d,k] * src[b,s,n], map[n,k])
// (convolution backward-input: s = Co, d = Ci; transposed forward: s = Ci, d = Co).
// One wavefront (= one workgroup) owns a row segment of 32 map pixels.  It keeps
// the source values of its pixels (64 source channels) in registers as MFMA B
// operands.  Destination channels are processed 16 at a time: per tap the 64x16
// weight slice is read straight from the packed weights (L1/L2 resident) as A
// operands and v_mfma_f32_16x16x4_f32 yields col[d][pixel] in registers.
//
// Scatter with LDS pre-reduction.  MFMA and ordinary vector instructions do not
// overlap on a SIMD here, and LDS float atomics retire about one lane every few
// cycles, so the scatter is built to need few instructions and no atomics:
//   * a pre-pass over the wave's map entries finds the bounding box of its
//     destination corners (rows x a circular interval of columns) - the wave's
//     private LDS window - and resolves every (pixel, tap, corner) ONCE into a
//     window slot (one byte) and a weight, cached in LDS for all channel blocks;
//   * the window is updated with plain 16-byte read-modify-writes (a lane's four
//     channels of one slot are adjacent).  That is race-free when the 16 lanes of an
//     instruction hit 16 different slots, which holds whenever the slots grow
//     strictly along the pixel row; the pre-pass checks exactly that per (tap,
//     corner) and marks the rare ones that fail, which go to global atomics, as do
//     waves whose box does not fit the window;
//   * after the taps of a group the window is flushed with one global atomic per
//     touched element (consecutive lanes, consecutive addresses) and cleared.
// Corners whose weight is exactly zero (integer coordinates) are skipped.
constexpr int kScDC = 16;        // destination channels per pass
constexpr int kScWaveWin = 160;  // window slots of a wave
constexpr int kScWinLd = 20;     // floats per slot: 16 channels + 4 of padding (bank spread)
constexpr int kScSC = 64;        // source channels per register block
constexpr int kScPx = 32;        // pixels per wave
constexpr int kScEntries = 40;   // cached (tap, point, corner) entries per pixel
constexpr int kScThreads = 64;

__device__ inline int wave_min(int v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v = min(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ inline int wave_max(int v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v = max(v, __shfl_xor(v, m, 64));
  return v;
}

// Column distance from a reference column on the circle of DW columns, in
// [-DW/2, DW/2): both arguments are in [0, DW), so one conditional add/sub wraps.
__device__ inline int circ_delta(int xx, int xref, int dw, int halfw) {
  int d = xx - xref;
  if (d >= dw - halfw) d -= dw;
  if (d < -halfw) d += dw;
  return d;
}

template <typename TD, int NCORN, int NP>
__global__ __launch_bounds__(kScThreads, 2) void product_scatter_mfma_kernel(
    const TD *__restrict__ src, const float *__restrict__ map, const float *__restrict__ iw,
    const float *__restrict__ wq, float *__restrict__ dst, int S, int D, int Spad, int DH, int DW,
    int MH, int MW, int K, int weighted, int wrap, int tiles_x, int tiles_per_img,
    const int *__restrict__ gate, int run_if_zero) {
  if (gate && ((*gate == 0) != (run_if_zero != 0))) return;  // device-side path selection
  constexpr int NE = NP * NCORN;           // cache entries per (pixel, tap)
  constexpr int TG = kScEntries / NE;      // taps per group (their entries fit the cache)
  static_assert(TG >= 1, "entry cache too small");
  __shared__ __attribute__((aligned(16))) float win[kScWaveWin][kScWinLd];  // [slot][channel]
  __shared__ float c_wt[TG * NE][kScPx];          // cached corner weights
  __shared__ unsigned char c_slot[TG * NE][kScPx];  // cached window slots, 255 = not cached
  __shared__ unsigned c_flag[TG][2];              // per tap: "any lane valid" / "needs atomics" bits

  const int lane = threadIdx.x;
  const int l15 = lane & 15, lq = lane >> 4;
  const int tile = xcd_contiguous_tile(blockIdx.x, gridDim.x);
  const int b = tile / tiles_per_img;
  const int t_in = tile - b * tiles_per_img;
  const int pi = t_in / tiles_x, j0 = (t_in - pi * tiles_x) * kScPx;
  const int N = MH * MW;
  const int64_t dplane = (int64_t)DH * DW;
  const int dchunks = (D + kScDC - 1) / kScDC;
  const int schunks = Spad / kScSC;
  const int halfw = DW >> 1;

  // ---- this lane's two pixels (MFMA column l15 of column blocks 0 and 1) -------
  int64_t npx[2];
  bool live[2];
#pragma unroll
  for (int nb = 0; nb < 2; nb++) {
    const int pj = j0 + nb * 16 + l15;
    live[nb] = pj < MW;
    npx[nb] = (int64_t)pi * MW + (live[nb] ? pj : j0);
  }

  // ---- pre-pass A: bounding box of the destination corners of the wave's pixels
  // (valid corners with a non-zero weight); the four 16-lane groups take every
  // fourth tap ------------------------------------------------------------------
  const int xref =
      wrap_index(to_int(floorf(map[((int64_t)pi * MW + j0) * K * NP * 2])), DW);
  int ymin = 0x7fffffff, ymax = -0x7fffffff, dmin = 0x7fffffff, dmax = -0x7fffffff;
  for (int k = lq; k < K; k += 4) {
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      if (!live[nb]) continue;
#pragma unroll
      for (int sp = 0; sp < NP; sp++) {
        const int64_t e = (npx[nb] * K + k) * NP + sp;
        CoordTap<NCORN> t;
        resolve_coords<NCORN>(map[e * 2], map[e * 2 + 1], DH, DW, wrap != 0,
                              weighted ? iw[e] : 1.f, t);
#pragma unroll
        for (int c = 0; c < NCORN; c++) {
          if ((t.ok & (1u << c)) && t.wt[c] != 0.f) {
            const int dx = circ_delta(t.xx[c], xref, DW, halfw);
            ymin = min(ymin, t.yy[c]);
            ymax = max(ymax, t.yy[c]);
            dmin = min(dmin, dx);
            dmax = max(dmax, dx);
          }
        }
      }
    }
  }
  ymin = wave_min(ymin);
  ymax = wave_max(ymax);
  dmin = wave_min(dmin);
  dmax = wave_max(dmax);
  if (ymin > ymax) return;  // nothing of this wave lands inside the destination
  const int ww = dmax - dmin + 1, wh = ymax - ymin + 1;
  const int wsz = ww * wh;
  const bool use_lds = wsz <= kScWaveWin;

  // global offsets of the window slots this lane flushes
  constexpr int kFlushRounds = (kScWaveWin + 63) / 64;
  int goff[kFlushRounds];
#pragma unroll
  for (int r = 0; r < kFlushRounds; r++) {
    const int slot = lane + r * 64;
    if (use_lds && slot < wsz) {
      const int wy = slot / ww, wx = slot - wy * ww;
      goff[r] = (ymin + wy) * DW + wrap_index(xref + dmin + wx, DW);
    } else {
      goff[r] = -1;
    }
  }
  for (int e = lane; e < kScWaveWin * kScWinLd; e += 64) (&win[0][0])[e] = 0.f;

  const TD *src_b = src + (int64_t)b * S * N;
  float *dst_b = dst + (int64_t)b * D * dplane;

  float breg[2][16];
  auto load_b = [&](int sc) {
#pragma unroll
    for (int nb = 0; nb < 2; nb++)
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int s = sc * kScSC + 4 * t + lq;
        breg[nb][t] = (live[nb] && s < S) ? to_f32(src_b[(int64_t)s * N + npx[nb]]) : 0.f;
      }
  };
  if (schunks == 1) load_b(0);

  // MFMA A operands: lane (l15, lq) of step t needs Wq[k][dc][sc*64 + 4t + lq][l15].
  const unsigned a_off = (unsigned)(lq * kScDC + l15) * 4u;
  auto load_a = [&](int dc, int k, int sc, float *reg) {
    const float *base = wq + (((int64_t)k * dchunks + dc) * Spad + sc * kScSC) * kScDC;  // uniform
#pragma unroll
    for (int t = 0; t < 16; t++) reg[t] = load_at(base + t * 4 * kScDC, a_off);
  };

  for (int k0 = 0; k0 < K; k0 += TG) {  // tap groups
    const int kn = min(TG, K - k0);
    // ---- pre-pass B: resolve the group's taps once into the LDS cache and decide,
    // per (tap, pixel block, point, corner), whether the plain window update is
    // race-free (valid lanes of the 16-lane group form one run of strictly
    // increasing slots; the four groups of an MFMA result hold different channels)
    for (int kb = 0; kb < kn; kb += 4) {  // uniform trip count: the ballots need every lane
      const int kl = kb + lq;  // tap within the group handled by this 16-lane group
      unsigned any_bits = 0, atom_bits = 0;
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
#pragma unroll
        for (int sp = 0; sp < NP; sp++) {
          CoordTap<NCORN> t;
          t.ok = 0;
          if (kl < kn && live[nb]) {
            const int64_t e = (npx[nb] * K + k0 + kl) * NP + sp;
            resolve_coords<NCORN>(map[e * 2], map[e * 2 + 1], DH, DW, wrap != 0,
                                  weighted ? iw[e] : 1.f, t);
          }
#pragma unroll
          for (int c = 0; c < NCORN; c++) {
            const bool valid = (t.ok & (1u << c)) && t.wt[c] != 0.f;
            const int slot =
                (valid && use_lds)
                    ? (t.yy[c] - ymin) * ww + circ_delta(t.xx[c], xref, DW, halfw) - dmin
                    : 0;
            const int prev = __shfl_up(slot, 1, 16);
            const int pvalid = __shfl_up((int)valid, 1, 16);
            const bool clash = valid && l15 > 0 && pvalid && slot <= prev;
            const unsigned m = (unsigned)((__ballot(valid) >> (16 * lq)) & 0xffffu);
            const unsigned cl = (unsigned)((__ballot(clash) >> (16 * lq)) & 0xffffu);
            const unsigned run = m ? (m >> __builtin_ctz(m)) : 0u;
            const bool atomics = !use_lds || cl != 0u || (run & (run + 1u)) != 0u;
            const int bit = (nb * NP + sp) * NCORN + c;
            if (m) any_bits |= 1u << bit;
            if (m && atomics) atom_bits |= 1u << bit;
            if (kl < kn) {
              const int row = kl * NE + sp * NCORN + c;
              c_slot[row][nb * 16 + l15] = (unsigned char)((valid && !atomics) ? slot : 255);
              c_wt[row][nb * 16 + l15] = valid ? t.wt[c] : 0.f;
            }
          }
        }
      }
      if (kl < kn && l15 == 0) {
        c_flag[kl][0] = any_bits;
        c_flag[kl][1] = atom_bits;
      }
    }
    __syncthreads();  // single-wave workgroup: orders the cache writes before its reads

    // ---- main loop over (destination-channel block, tap of the group, source block)
    const int units = dchunks * kn * schunks;
    float areg[2][16];
    load_a(0, k0, 0, areg[0]);
    int dc = 0, kl = 0, sc = 0;
    floatx4 acc[2];
    auto unit = [&](int u, float *acur, float *anext) {
      if (schunks > 1) load_b(sc);
      if (sc == 0) {
        acc[0] = floatx4{0.f, 0.f, 0.f, 0.f};
        acc[1] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
      const bool last_sc = sc + 1 == schunks;
      const int cdc = dc, ckl = kl;
      if (++sc == schunks) {
        sc = 0;
        if (++kl == kn) {
          kl = 0;
          ++dc;
        }
      }
      if (u + 1 < units) load_a(dc, k0 + kl, sc, anext);  // next unit's weights in flight
#pragma unroll
      for (int t = 0; t < 16; t++) {
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(acur[t], breg[0][t], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(acur[t], breg[1][t], acc[1], 0, 0, 0);
      }
      if (!last_sc) return;

      // scatter col[d = cdc*16 + lq*4 + i][pixel nb] through tap k0 + ckl
      const unsigned any_bits = c_flag[ckl][0], atom_bits = c_flag[ckl][1];
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
#pragma unroll
        for (int e = 0; e < NE; e++) {
          const int bit = nb * NE + e;
          if (!((any_bits >> bit) & 1u)) continue;  // uniform: no lane uses this corner
          const int row = ckl * NE + e;
          if (!((atom_bits >> bit) & 1u)) {
            const unsigned slot = c_slot[row][nb * 16 + l15];
            const float wt = c_wt[row][nb * 16 + l15];
            if (slot != 255u) {
              // one 16-byte read-modify-write: the lane's four channels are adjacent
              float4 *cell = reinterpret_cast<float4 *>(&win[slot][lq * 4]);
              float4 cur = *cell;
              cur.x += wt * acc[nb][0];
              cur.y += wt * acc[nb][1];
              cur.z += wt * acc[nb][2];
              cur.w += wt * acc[nb][3];
              *cell = cur;
            }
          } else if (live[nb]) {
            // rare: re-resolve this corner and use global atomics
            const int sp = e / NCORN, c = e % NCORN;
            const int64_t me = (npx[nb] * K + k0 + ckl) * NP + sp;
            CoordTap<NCORN> t;
            resolve_coords<NCORN>(map[me * 2], map[me * 2 + 1], DH, DW, wrap != 0,
                                  weighted ? iw[me] : 1.f, t);
            if ((t.ok & (1u << c)) && t.wt[c] != 0.f) {
              const int off = t.yy[c] * DW + t.xx[c];
#pragma unroll
              for (int i = 0; i < 4; i++) {
                const int d = cdc * kScDC + lq * 4 + i;
                if (d < D) atomic_add(dst_b + (int64_t)d * dplane + off, t.wt[c] * acc[nb][i]);
              }
            }
          }
        }
      }
      // after the last tap of the group: flush and clear the window
      if (use_lds && ckl == kn - 1) {
#pragma unroll
        for (int r = 0; r < kFlushRounds; r++) {
          if (goff[r] < 0) continue;
          const int slot = lane + r * 64;
          float vals[kScDC];
#pragma unroll
          for (int q = 0; q < kScDC / 4; q++) {
            float4 *cell = reinterpret_cast<float4 *>(&win[slot][q * 4]);
            const float4 cur = *cell;
            *cell = float4{0.f, 0.f, 0.f, 0.f};
            vals[q * 4 + 0] = cur.x;
            vals[q * 4 + 1] = cur.y;
            vals[q * 4 + 2] = cur.z;
            vals[q * 4 + 3] = cur.w;
          }
#pragma unroll
          for (int dl = 0; dl < kScDC; dl++) {
            const int d = cdc * kScDC + dl;
            if (vals[dl] != 0.f && d < D)
              atomic_add(dst_b + (int64_t)d * dplane + goff[r], vals[dl]);
          }
        }
      }
    };
    for (int u = 0; u < units; u += 2) {  // ping-pong the A operand registers
      unit(u, areg[0], areg[1]);
      if (u + 1 < units) unit(u + 1, areg[1], areg[0]);
    }
    __syncthreads();  // cache reads done before the next group's pre-pass rewrites it
  }
}

struct PixelTiling {
  int tw_shift, tiles_x, tiles_per_img;
  int64_t total;
};

// 2-D pixel tiles of 128: 4 x 32 when the map has at least 4 rows, else 1 x 128.  With 2-byte
// elements and wide images the tiles are 1 x 128 as well: a wave's 64 samples of a row then
// span 128 bytes instead of two runs of 64.
inline PixelTiling make_tiling(int64_t B, int64_t H, int64_t W, int elem) {
  PixelTiling t;
  t.tw_shift = H >= 4 ? 5 : 7;
  if (elem == 2 && W >= 256) t.tw_shift = 7;
  const int tw = 1 << t.tw_shift, th = kTilePx >> t.tw_shift;
  t.tiles_x = (int)((W + tw - 1) / tw);
  t.tiles_per_img = t.tiles_x * (int)((H + th - 1) / th);
  t.total = (int64_t)t.tiles_per_img * B;
  return t;
}

template <typename TD>
inline int weight_grad_ranges(int64_t total_tiles, int64_t A, int64_t G, int64_t K) {
  constexpr int kWgA = wg_plain_channels<TD>(), kWgCB = wg_gathered_blocks<TD>();
  const int64_t per_range = ((G + kWgCB * kGC - 1) / (kWgCB * kGC)) * ((A + kWgA - 1) / kWgA) *
                            ((K + kWgKT - 1) / kWgKT);
  int64_t r = std::max<int64_t>(8, (768 / per_range) / 8 * 8);  // about three workgroups per CU
  return (int)std::min<int64_t>(r, std::max<int64_t>(total_tiles, 1));
}

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

}  // namespace

// =================================================================================
// Host side.  Every launcher is a template on the storage type TD (float or bf16_t)
// and is instantiated for both at the end of the file.
// =================================================================================

bool mfma_supported(int64_t P) { return P >= 0 && P <= 4; }

namespace {

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct ModeArgs {
  int mode, weighted, wrap, np;
};
inline ModeArgs mode_args(int interp, int64_t P) {
  ModeArgs m;
  m.mode = canonical_interp(interp);
  m.weighted = P > 0 ? 1 : 0;
  m.wrap = m.mode == kInterpBispherical ? 1 : 0;
  m.np = P > 0 ? (int)P : 1;
  return m;
}

// Expands LAUNCH(NCORN, NP) for the interpolation mode and point count at hand.
#define MCX_DISPATCH_TAPS(m, LAUNCH)   \
  if ((m).mode == kInterpNearest) {    \
    switch ((m).np) {                  \
      case 1: LAUNCH(1, 1); break;     \
      case 2: LAUNCH(1, 2); break;     \
      case 3: LAUNCH(1, 3); break;     \
      default: LAUNCH(1, 4); break;    \
    }                                  \
  } else {                             \
    switch ((m).np) {                  \
      case 1: LAUNCH(4, 1); break;     \
      case 2: LAUNCH(4, 2); break;     \
      case 3: LAUNCH(4, 3); break;     \
      default: LAUNCH(4, 4); break;    \
    }                                  \
  }

// Channel-last staging of the source pays when neighbouring map entries point to unrelated
// source pixels; that is taken to be the case for single-row sources (mesh signals stored
// as [1, V] images) sampled with nearest interpolation.
inline bool use_channel_last(int64_t SH, int interp) {
  return SH == 1 && canonical_interp(interp) == kInterpNearest;
}
// Blocked staging ([B][Gpad/8][pixels][8]) of an image-like source: bf16 storage only.
inline bool use_channel_blocks(int64_t SH, int interp, size_t elem) {
  return elem == 2 && !use_channel_last(SH, interp) && SH > 1;
}
template <typename TD>
int launch_channel_blocks(const TD *src, TD *stage, int64_t B, int64_t G, int64_t plane,
                          hipStream_t s, const int *pair_mask = nullptr) {
  const int64_t Gpad = round_up(G, kGC);
  dim3 tg((unsigned)((plane + 255) / 256), (unsigned)(Gpad / 8), (unsigned)B);
  hipLaunchKernelGGL(to_channel_blocks_kernel<TD>, tg, dim3(256), 0, s, src, stage, (int)G, plane,
                     pair_mask);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

// `stage`: room for the channel-last copy (B * SH * SW * Gpad elements) when
// use_channel_last(SH, interp), unused otherwise.
template <typename TD>
int launch_gather_product(const TD *src, const float *map, const float *iw, const float *wp,
                          const TD *bias, TD *y, TD *stage, int64_t B, int64_t G, int64_t O,
                          int64_t SH, int64_t SW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                          int interp, const int *gate, int run_if_zero, hipStream_t s,
                          const float *addend = nullptr, bool staged = false,
                          const int *pair_mask = nullptr, bool packed_map = false,
                          bool accumulate = false, const int *row_mask = nullptr,
                          int mask_words = 1) {
  const int Opad = (int)round_up(O, kOT), Gpad = (int)round_up(G, kGC);
  const bool blocked = stage != nullptr && use_channel_blocks(SH, interp, sizeof(TD)) &&
                       SH * SW * 8 * (int64_t)sizeof(TD) <= 0xffffffffLL;
  const bool cl = blocked || (stage != nullptr && use_channel_last(SH, interp) &&
                              SH * SW * Gpad * (int64_t)sizeof(TD) <= 0xffffffffLL);
  if (cl && staged) {
    src = stage;  // the caller has made the copy already
  } else if (blocked) {
    if (int rc = launch_channel_blocks<TD>(src, stage, B, G, SH * SW, s)) return rc;
    src = stage;
  } else if (cl) {
    dim3 tg((unsigned)((SH * SW + 63) / 64), (unsigned)((Gpad + 63) / 64), (unsigned)B);
    hipLaunchKernelGGL(to_channel_last_kernel<TD>, tg, dim3(256), 0, s, src, stage, (int)G, Gpad,
                       SH * SW);
    MCX_HIP_CHECK_LAUNCH();
    src = stage;
  }
  const PixelTiling t = make_tiling(B, OH, OW, (int)sizeof(TD));
  if (t.total > 0x7fffffffLL) return MCX_E_SHAPE;
  // tap offsets are 32-bit byte offsets inside a source plane
  if (SH * SW * (int64_t)sizeof(TD) > 0xffffffffLL) return MCX_E_SHAPE;
  // bf16 storage with at least 128 output channels: 128 outputs per workgroup
  // (also fp32 over a channel-last source: a mesh signal's gather is a stream of unrelated
  // records from memory, which 128 outputs share instead of 64)
  const bool wide = Opad % (2 * kOT) == 0 && (sizeof(TD) == 2 || (cl && !blocked));
  if constexpr (sizeof(TD) == 2) {
    // bf16 images: the direct form, over pair words (taps straight from the map) or over
    // 8-channel blocks (entries of a packed map)
    // (a staged image and the packed weights are addressed as buffers of less than 4 GiB)
    const ModeArgs m0 = mode_args(interp, P);
    const bool from_map = blocked && !packed_map && m0.mode != kInterpNearest && m0.np == 1;
    const bool from_packed = blocked && packed_map && m0.mode == kInterpNearest &&
                             m0.np == 4;  // (the four entries of a packed map's cell)
    if ((from_map || from_packed) && !accumulate && OH * OW <= 0x7fffffffLL - kDgPx &&
        (int64_t)(Gpad / 8) * SH * SW * 16 < 0xffffff00LL &&
        K * (int64_t)(Gpad / kGC) * 2 * Opad * 16 < 0xffffff00LL) {
      const int64_t tiles_per_img = (OH * OW + kDgPx - 1) / kDgPx;
      if (tiles_per_img * B > 0x7fffffffLL) return MCX_E_SHAPE;
      const dim3 dgrid((unsigned)(tiles_per_img * B), (unsigned)(Opad / (wide ? 2 * kOT : kOT)));
#define MCX_LAUNCH_DIRECT(FORM, NA, OG, MASK, LEAD)                                              \
  hipLaunchKernelGGL((gather_product_bf16_direct_kernel<FORM, NA, OG>), dgrid, dim3(kThreads),   \
                     0, s, reinterpret_cast<const bf16_t *>(src), map, iw,                       \
                     reinterpret_cast<const uint16_t *>(wp),                                     \
                     reinterpret_cast<const bf16_t *>(bias), reinterpret_cast<bf16_t *>(y),      \
                     (int)O, Opad, Gpad, (int)SH, (int)SW, (int)(OH * OW), (int)OW, (int)K,      \
                     m0.weighted, m0.wrap, (int)tiles_per_img, gate, run_if_zero, addend, MASK,  \
                     LEAD, row_mask, mask_words)
#define MCX_LAUNCH_DIRECT_NA(FORM, OG)                                  \
  if (pair_mask) {                                                      \
    MCX_LAUNCH_DIRECT(FORM, 2, OG, pair_mask, 1);                       \
    MCX_LAUNCH_DIRECT(FORM, 4, OG, pair_mask, 0);                       \
  } else {                                                              \
    MCX_LAUNCH_DIRECT(FORM, 4, OG, (const int *)nullptr, 0);            \
  }
      profile_begin(s);
      if (from_map) {
        if (wide) {
          MCX_LAUNCH_DIRECT_NA(false, 2)
        } else {
          MCX_LAUNCH_DIRECT_NA(false, 1)
        }
      } else {
        if (wide) {
          MCX_LAUNCH_DIRECT_NA(true, 2)
        } else {
          MCX_LAUNCH_DIRECT_NA(true, 1)
        }
      }
      profile_end(s);
#undef MCX_LAUNCH_DIRECT_NA
#undef MCX_LAUNCH_DIRECT
      MCX_HIP_CHECK_LAUNCH();
      return 0;
    }
  }
  dim3 grid((unsigned)t.total, (unsigned)(Opad / (wide ? 2 * kOT : kOT)));
  const ModeArgs m = mode_args(interp, P);
  // `pair_mask` (four-pair taps only): launch the two-pair form as well; the mask picks one
#define MCX_LAUNCH_NA(NCORN, NP, OG, CL, NA, MASK, LEAD)                                         \
  hipLaunchKernelGGL((gather_product_mfma_kernel<TD, NCORN, NP, OG, CL, NA>), grid,              \
                     dim3(kThreads), 0, s, src, map, iw, wp, bias, y, (int)G, (int)O, Opad,      \
                     Gpad, (int)SH, (int)SW, (int)OH, (int)OW, (int)K, m.weighted, m.wrap,       \
                     t.tiles_x, t.tiles_per_img, t.tw_shift, gate, run_if_zero, addend, MASK,    \
                     LEAD, packed_map ? 1 : 0, accumulate ? 1 : 0, blocked ? 1 : 0, row_mask,     \
                     mask_words)
#define MCX_LAUNCH_CL(NCORN, NP, OG, CL)                                      \
  if constexpr (NCORN * NP == 4) {                                            \
    if (pair_mask) {                                                          \
      MCX_LAUNCH_NA(NCORN, NP, OG, CL, 2, pair_mask, 1);                      \
      MCX_LAUNCH_NA(NCORN, NP, OG, CL, NCORN * NP, pair_mask, 0);             \
    } else {                                                                  \
      MCX_LAUNCH_NA(NCORN, NP, OG, CL, NCORN * NP, (const int *)nullptr, 0);  \
    }                                                                         \
  } else {                                                                    \
    MCX_LAUNCH_NA(NCORN, NP, OG, CL, NCORN * NP, (const int *)nullptr, 0);    \
  }
#define MCX_LAUNCH_OG(NCORN, NP, OG)           \
  if constexpr (NCORN == 1 || sizeof(TD) == 2) { \
    if (cl) {                                  \
      MCX_LAUNCH_CL(NCORN, NP, OG, true);      \
    } else {                                   \
      MCX_LAUNCH_CL(NCORN, NP, OG, false);     \
    }                                          \
  } else {                                     \
    MCX_LAUNCH_CL(NCORN, NP, OG, false);       \
  }
#define MCX_LAUNCH(NCORN, NP)                               \
  if constexpr (sizeof(TD) == 2 || NCORN == 1) {            \
    if (wide) {                                             \
      MCX_LAUNCH_OG(NCORN, NP, 2);                          \
    } else {                                                \
      MCX_LAUNCH_OG(NCORN, NP, 1);                          \
    }                                                       \
  } else {                                                  \
    MCX_LAUNCH_OG(NCORN, NP, 1);                            \
  }
  profile_begin(s);
  MCX_DISPATCH_TAPS(m, MCX_LAUNCH)
  profile_end(s);
#undef MCX_LAUNCH
#undef MCX_LAUNCH_OG
#undef MCX_LAUNCH_CL
#undef MCX_LAUNCH_NA
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

// Maps of up to kSmallMapEntries (location, tap) entries have their pair mask made on the
// weight-packing launch of a forward call (a word per block, see PairMaskJob); elsewhere a map
// of up to kTinyMapEntries gets a launch of one block, which needs no clearing launch before it.
constexpr int64_t kSmallMapEntries = 262144;
constexpr int64_t kTinyMapEntries = 4096;

template <typename TD>
int launch_pack_weights(const TD *w, float *wp, int64_t O, int64_t G, int64_t K, int transposed,
                        hipStream_t s, int *clear = nullptr, ZeroJob zero = ZeroJob{nullptr, 0},
                        PairMaskJob pm = PairMaskJob{}) {
  const int Opad = (int)round_up(O, kOT), Gpad = (int)round_up(G, kGC);
  const int64_t packed = (int64_t)K * Gpad * Opad;
  // (bf16 storage: the bf16 MFMA operand layout in the same scratch, half the bytes)
  const int64_t work = std::max(packed, zero.count * 4);
  const dim3 grid((unsigned)std::min<int64_t>((work + 255) / 256, 4096) +
                  (pm.mask ? (unsigned)pm.blocks : 0u));
  hipLaunchKernelGGL(pack_weights_kernel<TD>, grid, dim3(256), 0, s, w, (void *)wp, (int)O, (int)G,
                     (int)K, Opad, Gpad, transposed, clear, zero, pm);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

inline PairMaskJob pair_mask_job(const float *map, const float *iw, int *mask, const ModeArgs &m,
                                 int64_t GH, int64_t GW, int64_t samples) {
  // (a block of 256 threads per 2048 entries, 64 at most: the readers load a word per lane)
  const int blocks = (int)std::min<int64_t>(64, (samples + 2047) / 2048);
  return PairMaskJob{map, iw, mask, blocks, m.np, m.weighted, m.wrap, (int)GH, (int)GW,
                     m.mode == kInterpNearest ? 1 : 4, samples};
}

// mask[0] >= 4 iff the map uses a pair beyond the first two of a tap.
// `cleared`: an earlier kernel on the stream has zeroed the mask.
int launch_pair_mask(const float *map, const float *iw, int *mask, const ModeArgs &m, int64_t GH,
                     int64_t GW, int64_t samples, hipStream_t s, bool cleared = false) {
  const bool small = samples <= kTinyMapEntries;  // one block, which stores the word outright
  if (!cleared && !small)
    if (int rc = fill_f32((float *)mask, 1, 0.f, s)) return rc;
  const dim3 mg(small ? 1u : (unsigned)std::min<int64_t>((samples + 255) / 256, 2048));
  const dim3 threads(small ? 1024 : 256);
  if (m.mode == kInterpNearest)
    hipLaunchKernelGGL(map_pair_mask_kernel<1>, mg, threads, 0, s, map, iw, mask, m.np,
                       m.weighted, m.wrap, (int)GH, (int)GW, samples);
  else
    hipLaunchKernelGGL(map_pair_mask_kernel<4>, mg, threads, 0, s, map, iw, mask, m.np,
                       m.weighted, m.wrap, (int)GH, (int)GW, samples);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

}  // namespace

// (defined with the map plans below)
namespace {
constexpr int kPlanSlots = 4;  // resolved entries per (location, tap) of a plan's gather part
bool gather_plan_applies(int interp, int64_t P);
template <int NCORN>
__global__ void build_gather_plan_kernel(const float *__restrict__ map,
                                         const float *__restrict__ iw, float2 *__restrict__ gmap,
                                         int np, int weighted, int wrap, int SH, int SW, int K,
                                         int64_t total);
// bf16 images under single-point bilinear taps: a forward call without a plan resolves the
// taps once into the same form before its product (a tenth of a millisecond where the product
// kernel would spend four resolving them tile by tile)
inline bool resolves_per_call(size_t elem, int64_t SH, int interp, int64_t P, int64_t MH,
                              int64_t MW, int64_t K) {
  return elem == 2 && SH > 1 && canonical_interp(interp) != kInterpNearest && P <= 1 &&
         MH * MW * K * kPlanSlots * 2 <= 0x7fffffffLL;
}
}  // namespace
size_t mfma_gather_plan_offset(int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,
                               int64_t P);

// ---- gather-product --------------------------------------------------------------
// Packed weights, then (single-row sources) the channel-last copy of the source, sized
// for 4-byte elements.
size_t mfma_gather_product_bytes(int64_t O, int64_t G, int64_t K, int64_t B, int64_t SH,
                                 int64_t SW, int elem, int64_t MH, int64_t MW) {
  size_t n = align256((size_t)(K * round_up(G, kGC) * round_up(O, kOT)) * sizeof(float));
  n += 256;  // the map's pair mask
  if (SH == 1 || elem == 2)
    n += align256((size_t)(B * SH * SW * round_up(G, kGC)) * sizeof(float));
  // the taps resolved per call (whatever the interpolation will be: it is not known here)
  if (resolves_per_call((size_t)elem, SH, kInterpBilinear, 1, MH, MW, K))
    n += align256((size_t)(MH * MW * K) * kPlanSlots * sizeof(float2));
  return n;
}

// scratch: mfma_gather_product_bytes(...) bytes.
template <typename TD>
int mfma_gather_product(const TD *src, const float *map, const float *iw, const TD *w,
                        const TD *bias, TD *y, void *scratch, int64_t B, int64_t G, int64_t O,
                        int64_t SH, int64_t SW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                        int interp, hipStream_t s, const void *plan) {
  float *wp = (float *)scratch;
  // (fp32 images with four-corner taps: resolving the taps in the kernel and reading them
  // resolved measured the same within 1 %, so there only the plan's pair mask is used and the
  // 32 bytes per tap of the resolved form are not read; single-row sources and bf16 storage
  // gain from the resolved form)
  const bool resolved_pays =
      !(SH > 1 && canonical_interp(interp) != kInterpNearest && sizeof(TD) == 4);
  if (plan && resolved_pays && gather_plan_applies(interp, P) &&
      OH * OW * K * kPlanSlots * 2 <= 0x7fffffffLL) {
    // the map's taps were resolved when the plan was built: read them as four pre-resolved
    // pairs per tap; flag word 4 of the plan says whether only the first two are ever in use
    const char *pb = (const char *)plan;
    const float *gmap = (const float *)(pb + mfma_gather_plan_offset(SH, SW, OH, OW, K, P));
    const int *flags = (const int *)plan + SH * SW * K;
    TD *stage = (SH == 1 || sizeof(TD) == 2)
                    ? reinterpret_cast<TD *>((char *)scratch + 256 +
                                             align256((size_t)(K * round_up(G, kGC) *
                                                               round_up(O, kOT)) * 4))
                    : nullptr;
    if (int rc = launch_pack_weights<TD>(w, wp, O, G, K, 0, s)) return rc;
    const ModeArgs pm = mode_args(interp, P);
    const bool four_pairs = pm.np * (pm.mode == kInterpNearest ? 1 : 4) == 4;
    return launch_gather_product<TD>(src, gmap, nullptr, wp, bias, y, stage, B, G, O, SH, SW, OH,
                                     OW, K, kPlanSlots, kInterpNearest, nullptr, 0, s, nullptr,
                                     false, four_pairs ? flags + 4 : nullptr, true);
  }
  int *pair_mask = reinterpret_cast<int *>(
      (char *)scratch + align256((size_t)(K * round_up(G, kGC) * round_up(O, kOT)) * 4));
  TD *stage = (SH == 1 || sizeof(TD) == 2) ? reinterpret_cast<TD *>((char *)pair_mask + 256)
                                           : nullptr;
  const ModeArgs m = mode_args(interp, P);
  const bool four_pairs = m.np * (m.mode == kInterpNearest ? 1 : 4) == 4;
  if (!plan && resolves_per_call(sizeof(TD), SH, interp, P, OH, OW, K)) {
    float2 *gmap = reinterpret_cast<float2 *>(
        (char *)stage + align256((size_t)(B * SH * SW * round_up(G, kGC)) * sizeof(float)));
    if (int rc = launch_pack_weights<TD>(w, wp, O, G, K, 0, s, pair_mask)) return rc;
    if (int rc = launch_pair_mask(map, iw, pair_mask, m, SH, SW, OH * OW * K, s, true)) return rc;
    const int64_t total = OH * OW * K;
    hipLaunchKernelGGL(build_gather_plan_kernel<4>,
                       dim3((unsigned)(((OH * OW + 63) / 64 * 64 * K + 255) / 256)), dim3(256), 0,
                       s, map, iw, gmap, m.np, m.weighted, m.wrap, (int)SH, (int)SW, (int)K,
                       total);
    MCX_HIP_CHECK_LAUNCH();
    return launch_gather_product<TD>(src, reinterpret_cast<const float *>(gmap), nullptr, wp, bias,
                                     y, stage, B, G, O, SH, SW, OH, OW, K, kPlanSlots,
                                     kInterpNearest, nullptr, 0, s, nullptr, false, pair_mask,
                                     true);
  }
  const int *mask = pair_mask;
  // the pair mask of a small map is made by the last block of the packing launch
  const bool mask_on_pack = four_pairs && !plan && OH * OW * K <= kSmallMapEntries;
  if (int rc = launch_pack_weights<TD>(
          w, wp, O, G, K, 0, s, mask_on_pack ? nullptr : pair_mask, ZeroJob{nullptr, 0},
          mask_on_pack ? pair_mask_job(map, iw, pair_mask, m, SH, SW, OH * OW * K)
                       : PairMaskJob{}))
    return rc;
  if (four_pairs) {
    if (plan)  // flag word 4 of a plan built for this map
      mask = (const int *)plan + SH * SW * K + 4;
    else if (!mask_on_pack)
      if (int rc = launch_pair_mask(map, iw, pair_mask, m, SH, SW, OH * OW * K, s, true))
        return rc;
  }
  const PairMaskJob job = mask_on_pack ? pair_mask_job(map, iw, pair_mask, m, SH, SW, OH * OW * K)
                                       : PairMaskJob{};
  return launch_gather_product<TD>(src, map, iw, wp, bias, y, stage, B, G, O, SH, SW, OH, OW, K,
                                   P, interp, nullptr, 0, s, nullptr, false,
                                   four_pairs ? mask : nullptr, false, false, nullptr,
                                   mask_on_pack ? job.blocks : 1);
}

// ---- weight gradient ---------------------------------------------------------------
// Per-range partial sums of gW, per-range partial sums of the plain operand, then
// (single-row gathered operands) their channel-last copy.
size_t mfma_weight_grad_bytes(int64_t B, int64_t A, int64_t G, int64_t MH, int64_t MW, int64_t K,
                              int64_t GH, int64_t GW, size_t elem) {
  // (the tiling and the number of ranges depend on the storage type and on the kernel)
  size_t ranges =
      (size_t)std::max(weight_grad_ranges<float>(make_tiling(B, MH, MW, 4).total, A, G, K),
                       weight_grad_ranges<bf16_t>(make_tiling(B, MH, MW, 2).total, A, G, K));
  if (elem == 2)
    ranges = std::max(
        ranges, (size_t)ring_weight_grad_ranges(make_tiling(B, MH, MW, 2).total, A, G, K));
  size_t n = align256(ranges * (size_t)(round_up(A, 4) * G * K) * sizeof(float));
  n += align256(ranges * (size_t)A * sizeof(float));
  n += 256;  // the map's pair mask
  // a copy of the gathered operand: channel-last for single-row sources, in blocks of 8
  // channels for bf16 images
  if (GH == 1)
    n += align256((size_t)(B * GH * GW * round_up(G, kGC)) * sizeof(float));
  else if (elem == 2)
    n += align256((size_t)(B * GH * GW * round_up(G, kGC)) * elem);
  else  // fp32 images: the table of resolved two-pair taps (resolve_tap_table_kernel)
    n += align256((size_t)make_tiling(B, MH, MW, 4).tiles_per_img * (size_t)K * kTilePx * 16);
  // bf16 images: the plain operand as MFMA fragments per pixel tile (to_plain_fragments_kernel)
  // and the table of resolved taps (resolve_tap_table_kernel, four pairs per tap at most)
  if (GH > 1 && elem == 2) {
    const size_t tiles = (size_t)make_tiling(B, MH, MW, 2).total;
    n += align256(tiles * (size_t)round_up(A, 32) * kTilePx * elem);
    n += align256((size_t)make_tiling(B, MH, MW, 2).tiles_per_img * (size_t)K * kTilePx * 8 *
                  sizeof(unsigned));
  }
  return n;
}

// scratch: mfma_weight_grad_bytes(...) bytes.  plain_sum (may be NULL): [A], receives the
// sum of the plain operand over images and pixels (a convolution's bias gradient).
template <typename TD>
int mfma_weight_grad(const TD *plain, const TD *gath, const float *map, const float *iw, TD *gw,
                     void *scratch, int64_t B, int64_t A, int64_t G, int64_t GH, int64_t GW,
                     int64_t MH, int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                     TD *plain_sum, const void *plan) {
  float *part = (float *)scratch;
  const PixelTiling t = make_tiling(B, MH, MW, (int)sizeof(TD));
  if (t.total > 0x7fffffffLL) return MCX_E_SHAPE;
  if (GH * GW * (int64_t)sizeof(TD) > 0xffffffffLL) return MCX_E_SHAPE;  // 32-bit tap offsets
  constexpr int kWgA = wg_plain_channels<TD>(), kWgCB = wg_gathered_blocks<TD>();
  const ModeArgs m = mode_args(interp, P);
  const int cgroups = (int)((G + kWgCB * kGC - 1) / (kWgCB * kGC));
  const int64_t Gpad = round_up(G, kGC);
  const bool cl = use_channel_last(GH, interp) &&
                  GH * GW * Gpad * (int64_t)sizeof(TD) <= 0xffffffffLL;
  // bf16 images under unweighted bilinear taps: the ring kernel, in its two-pair form for maps
  // whose lower corners weigh nothing and its four-pair form for the others (the pair mask
  // lets one of the two launches run)
  // (its 16-byte pieces of the plain operand want rows that are a multiple of 8 pixels, and
  // an image of either operand is addressed as a buffer of less than 4 GiB)
  const bool ring = sizeof(TD) == 2 && !cl && GH > 1 && m.np == 1 && m.mode != kInterpNearest &&
                    GH * GW * 16 < 0xffffff00LL && MW % 8 == 0 &&
                    (reinterpret_cast<uintptr_t>(plain) & 15) == 0 && B <= 65535 &&
                    A <= 32 * 65535;
  const int ranges = ring ? ring_weight_grad_ranges(t.total, A, G, K)
                          : weight_grad_ranges<TD>(t.total, A, G, K);
  float *sum_part = reinterpret_cast<float *>(
      (char *)scratch + align256((size_t)ranges * (size_t)(round_up(A, 4) * G * K) * 4));
  int *pair_mask = reinterpret_cast<int *>((char *)sum_part + align256((size_t)ranges * A * 4));
  int *const pair_mask_ws = pair_mask;  // (a plan may supply the mask; the copy's room follows this one)
  if (cl) {
    TD *stage = reinterpret_cast<TD *>((char *)pair_mask + 256);
    dim3 tg((unsigned)((GH * GW + 63) / 64), (unsigned)((Gpad + 63) / 64), (unsigned)B);
    hipLaunchKernelGGL(to_channel_last_kernel<TD>, tg, dim3(256), 0, s, gath, stage, (int)G,
                       (int)Gpad, GH * GW);
    MCX_HIP_CHECK_LAUNCH();
    gath = stage;
  }
  dim3 grid((unsigned)(ranges * cgroups), (unsigned)((A + kWgA - 1) / kWgA),
            (unsigned)((K + kWgKT - 1) / kWgKT));
  // Four pairs per tap: it pays to find out (on the device) whether only the first two pairs
  // are ever in use (bilinear maps with integral rows, two of four points weighted) and to
  // launch both variants, of which one returns at once.
  const bool two_variants = m.np * (m.mode == kInterpNearest ? 1 : 4) == 4;
  if (two_variants) {
    if (plan)  // flag word 4 of a plan built for this map (see mfma_scatter_plan_build)
      pair_mask = (int *)const_cast<void *>(plan) + GH * GW * K + 4;
    else if (int rc = launch_pair_mask(map, iw, pair_mask, m, GH, GW, MH * MW * K, s))
      return rc;
  }
  // fp32 images under single-point bilinear taps: the taps of the two-pair form resolved once
  // (the table follows the pair mask in the scratch)
  const uint4 *tap_table = nullptr;
  if (sizeof(TD) == 4 && !cl && GH > 1 && m.np == 1 && m.mode != kInterpNearest && two_variants) {
    unsigned *table = reinterpret_cast<unsigned *>((char *)pair_mask_ws + 256);
    hipLaunchKernelGGL((resolve_tap_table_kernel<2, 4, false>), dim3((unsigned)t.tiles_per_img),
                       dim3(256), 0, s, map, table, (int)GH, (int)GW, (int)MH, (int)MW, (int)K,
                       m.wrap, t.tiles_x, t.tw_shift, pair_mask);
    MCX_HIP_CHECK_LAUNCH();
    tap_table = reinterpret_cast<const uint4 *>(table);
  }
#define MCX_LAUNCH_NA(NCORN, NP, CL, NA, MASK, LEAD)                                             \
  hipLaunchKernelGGL((weight_grad_mfma_kernel<TD, NCORN, NP, CL, NA>), grid, dim3(kThreads), 0,  \
                     s, plain, gath, map, iw, part, (int)A, (int)G, (int)GH, (int)GW, (int)MH,   \
                     (int)MW, (int)K, m.weighted, m.wrap, t.tiles_x, t.tiles_per_img,            \
                     t.tw_shift, (int)t.total, ranges, cgroups,                                  \
                     plain_sum ? sum_part : (float *)nullptr, MASK, LEAD, tap_table)
#define MCX_LAUNCH_CL(NCORN, NP, CL)                                          \
  if constexpr (NCORN * NP == 4) {                                            \
    if (!ring) {                                                              \
      MCX_LAUNCH_NA(NCORN, NP, CL, 2, pair_mask, 1);                          \
      MCX_LAUNCH_NA(NCORN, NP, CL, NCORN * NP, pair_mask, 0);                 \
    }                                                                         \
  } else {                                                                    \
    MCX_LAUNCH_NA(NCORN, NP, CL, NCORN * NP, (const int *)nullptr, 0);        \
  }
#define MCX_LAUNCH(NCORN, NP)              \
  if constexpr (NCORN == 1) {              \
    if (cl) {                              \
      MCX_LAUNCH_CL(NCORN, NP, true);      \
    } else {                               \
      MCX_LAUNCH_CL(NCORN, NP, false);     \
    }                                      \
  } else {                                 \
    MCX_LAUNCH_CL(NCORN, NP, false);       \
  }
  if constexpr (sizeof(TD) == 2) {
    if (ring) {
      TD *stage = reinterpret_cast<TD *>((char *)pair_mask_ws + 256);
      if (int rc = launch_channel_blocks<TD>(gath, stage, B, G, GH * GW, s)) return rc;
      // the plain operand tile by tile, after the blocks of the gathered one
      bf16_t *tiles = reinterpret_cast<bf16_t *>(
          (char *)stage + align256((size_t)(B * GH * GW * Gpad) * sizeof(TD)));
      hipLaunchKernelGGL(to_plain_fragments_kernel,
                         dim3((unsigned)((t.tiles_per_img + kFragTiles - 1) / kFragTiles),
                              (unsigned)((A + 31) / 32), (unsigned)B),
                         dim3(256), 0, s, reinterpret_cast<const bf16_t *>(plain), tiles, (int)A,
                         (int)MH, (int)MW, t.tiles_x, t.tiles_per_img, t.tw_shift);
      MCX_HIP_CHECK_LAUNCH();
      // the taps, resolved once for all workgroups (two or four pairs: the mask decides)
      unsigned *table = reinterpret_cast<unsigned *>(
          (char *)tiles + align256((size_t)t.total * (size_t)round_up(A, 32) * kTilePx * sizeof(TD)));
      const dim3 rgrid((unsigned)t.tiles_per_img);
      hipLaunchKernelGGL((resolve_tap_table_kernel<2, 16, true>), rgrid, dim3(256), 0, s, map, table, (int)GH,
                         (int)GW, (int)MH, (int)MW, (int)K, m.wrap, t.tiles_x, t.tw_shift,
                         pair_mask);
      hipLaunchKernelGGL((resolve_tap_table_kernel<4, 16, true>), rgrid, dim3(256), 0, s, map, table, (int)GH,
                         (int)GW, (int)MH, (int)MW, (int)K, m.wrap, t.tiles_x, t.tw_shift,
                         pair_mask);
      MCX_HIP_CHECK_LAUNCH();
    }
  }
  profile_begin(s);
  if constexpr (sizeof(TD) == 2) {
    if (ring) {
      const int rg_groups = (int)((G + kRgG - 1) / kRgG), rg_passes = (int)((K + kRgKT - 1) / kRgKT);
#define MCX_LAUNCH_RING(NA)                                                                       \
  hipLaunchKernelGGL(weight_grad_bf16_ring_kernel<NA>,                                            \
                     dim3((unsigned)(ranges * rg_groups * rg_passes),                             \
                          (unsigned)((A + kRgA - 1) / kRgA)),                                     \
                     dim3(kThreads), 0, s,                                                        \
                     reinterpret_cast<const TD *>(                                                \
                         (char *)pair_mask_ws + 256 +                                             \
                         align256((size_t)(B * GH * GW * Gpad) * sizeof(TD))),                    \
                     reinterpret_cast<const TD *>((char *)pair_mask_ws + 256),                    \
                     reinterpret_cast<const unsigned *>(                                          \
                         (char *)pair_mask_ws + 256 +                                             \
                         align256((size_t)(B * GH * GW * Gpad) * sizeof(TD)) +                    \
                         align256((size_t)t.total * (size_t)round_up(A, 32) * kTilePx *           \
                                  sizeof(TD))),                                                   \
                     part, (int)A, (int)G, (int)Gpad, (int)GH, (int)GW, (int)K, t.tiles_per_img,  \
                     (int)t.total, ranges, rg_groups, rg_passes,                                  \
                     plain_sum ? sum_part : (float *)nullptr, pair_mask)
      MCX_LAUNCH_RING(2);
      MCX_LAUNCH_RING(4);
#undef MCX_LAUNCH_RING
      MCX_HIP_CHECK_LAUNCH();
    }
  }
  MCX_DISPATCH_TAPS(m, MCX_LAUNCH)
  profile_end(s);
#undef MCX_LAUNCH
#undef MCX_LAUNCH_NA
#undef MCX_LAUNCH_CL
  MCX_HIP_CHECK_LAUNCH();
  const int64_t n = round_up(A, 4) * G * K;
  const int64_t n2 = plain_sum ? A : 0;
  hipLaunchKernelGGL(reduce_partials_kernel<TD>, dim3((unsigned)((n + 63) / 64 + (n2 + 63) / 64)),
                     dim3(64, 4), 0, s, part, gw, (int)A, (int)round_up(A, 4), (int)G, (int)K,
                     sum_part, plain_sum, n2, ranges);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

// ---- product-scatter ---------------------------------------------------------------
namespace {

// Transposed map.  A scatter through map[n,k] is a gather through the transposed
// map: destination pixel p receives wt * col[., k, n] from every (n, corner) that
// lands on it.  When no (p, k) receives more than kTransSlots contributions (true for
// resolution-preserving maps such as the latitude-distorted kernels), the product-
// scatter equals a weighted, nearest-neighbour gather-product over the transposed
// map, which needs no atomics at all and reuses the forward kernel.  This kernel
// builds that map: tmap[k][slot][p] = (index of source pixel n as bits, corner weight);
// a slot counter per (k, p) hands out slots and an overflow flag selects the scatter
// kernel instead (both kernels are always enqueued; the flag gates them on the device).
// A wave takes 64 consecutive map pixels of one tap: under an image-like map they land on
// neighbouring destination pixels, so its counter updates and slot writes fall into a few
// cache lines (counters are [tap][pixel] like the slots); the taps of a run of pixels are
// neighbouring waves, which read the same lines of the map.
constexpr int kTransSlots = 4;
constexpr int kTransSlotsConst = kTransSlots;

// A contribution that finds its cell full goes to the overflow list (destination pixel,
// source pixel, tap, weight), applied afterwards with atomics by overflow_scatter_kernel;
// only when that list is full too (or there is none) the flag sends the whole product to
// the scatter kernel.
struct OverflowEntry {
  int p, n, k;
  float wt;
};

template <int NCORN>
__global__ void build_transposed_map_kernel(const float *__restrict__ map,
                                            const float *__restrict__ iw, int *__restrict__ cnt,
                                            float2 *__restrict__ tmap, float2 *__restrict__ tmap2,
                                            int *__restrict__ overflow,
                                            OverflowEntry *__restrict__ ovf, int ovf_cap, int np,
                                            int weighted, int wrap, int DH, int DW, int MW, int K,
                                            int64_t pixels) {
  const int64_t t0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t run = t0 / (64 * (int64_t)K);  // 64 map pixels x K taps
  const int r = (int)(t0 - run * 64 * K);
  const int k = r >> 6;
  const int64_t n = run * 64 + (r & 63);
  if (n >= pixels) return;
  const int64_t e = n * K + k;
  const int64_t DHW = (int64_t)DH * DW;
  const float nbits = __builtin_bit_cast(float, (int)n);
  for (int sp = 0; sp < np; sp++) {
    const int64_t m = e * np + sp;
    CoordTap<NCORN> t;
    resolve_coords<NCORN>(map[m * 2], map[m * 2 + 1], DH, DW, wrap != 0, weighted ? iw[m] : 1.f,
                          t);
#pragma unroll
    for (int c = 0; c < NCORN; c++) {
      if (!(t.ok & (1u << c)) || t.wt[c] == 0.f) continue;
      const int64_t pix = (int64_t)t.yy[c] * DW + t.xx[c];
      const int64_t cell = (int64_t)k * DHW + pix;
      const int slot = atomicAdd(&cnt[cell], 1);
      // slots are stored [tap][slot][pixel] (see the gather-product kernel's packed maps)
      if (slot < kTransSlots) {
        tmap[((int64_t)k * kTransSlots + slot) * DHW + pix] = make_float2(nbits, t.wt[c]);
      } else if (tmap2 && slot < 2 * kTransSlots) {  // second level (a second gather pass)
        tmap2[((int64_t)k * kTransSlots + slot - kTransSlots) * DHW + pix] =
            make_float2(nbits, t.wt[c]);
      } else {
        // overflow[0]: flag, overflow[1]: length of the overflow list
        const int pos = ovf_cap > 0 ? atomicAdd(&overflow[1], 1) : 0;
        if (pos < ovf_cap)
          ovf[pos] = OverflowEntry{t.yy[c] * DW + t.xx[c], (int)n, k, t.wt[c]};
        else
          overflow[0] = 1;  // benign race: every writer stores the same value
      }
    }
  }
}

// accum[b, d, p] += wt * sum_s W[s, d, k] * src[b, s, n] for every overflow entry: one wave
// per (entry, image), a lane per destination channel.  `wp` holds the weights in the
// gather-product's packed layout (fp32: Wp[k][s][d]; bf16: Wb[k][chunk][kg][d][8]); `src_cl`,
// when not null, is the channel-last copy [B][MN][Spad] of the source, else src is
// [B][S][MN].  `accum` is a channel-last fp32 image [B][DN][Dpad] (a wave's 64 atomics fall
// into two cache lines instead of 64) that the gather's epilogue adds.  A fixed grid walks
// the list, so an empty list costs one launch of idle workgroups.
template <typename TD>
__global__ __launch_bounds__(64) void overflow_scatter_kernel(
    const TD *__restrict__ src, const TD *__restrict__ src_cl, const void *__restrict__ wp,
    float *__restrict__ accum, const OverflowEntry *__restrict__ ovf,
    const int *__restrict__ overflow, int ovf_cap, int S, int Spad, int D, int Dpad, int64_t MN,
    int64_t DN) {
  if (overflow[0] != 0) return;  // the scatter kernel does the whole product
  const int count = min(overflow[1], ovf_cap);
  const int b = blockIdx.y, lane = threadIdx.x;
  const int chunks = Spad / kGC;
  for (int e = blockIdx.x; e < count; e += gridDim.x) {
    const OverflowEntry en = ovf[e];
    for (int d0 = 0; d0 < D; d0 += 64) {
      const int d = min(d0 + lane, Dpad - 1);
      float acc = 0.f;
      for (int s8 = 0; s8 < Spad / 8; s8++) {  // 8 source channels at a time (both are padded)
        float x[8], wv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const int sc = s8 * 8 + j;
          x[j] = src_cl ? to_f32(src_cl[((int64_t)b * MN + en.n) * Spad + sc])
                        : (sc < S ? to_f32(src[((int64_t)b * S + sc) * MN + en.n]) : 0.f);
        }
        if constexpr (sizeof(TD) == 2) {
          const int64_t wi = ((((int64_t)en.k * chunks + (s8 >> 1)) * 2 + (s8 & 1)) * Dpad + d) << 3;
          const uint4 q = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(wp) + wi);
          const unsigned w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int j = 0; j < 4; j++) {
            wv[2 * j] = __builtin_bit_cast(float, w4[j] << 16);
            wv[2 * j + 1] = __builtin_bit_cast(float, w4[j] & 0xffff0000u);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; j++)
            wv[j] = reinterpret_cast<const float *>(wp)[((int64_t)en.k * Spad + s8 * 8 + j) * Dpad + d];
        }
#pragma unroll
        for (int j = 0; j < 8; j++) acc = __builtin_fmaf(x[j], wv[j], acc);
      }
      if (d0 + lane < D) atomic_add(accum + ((int64_t)b * DN + en.p) * Dpad + d, en.wt * acc);
    }
  }
}

// Two jobs that follow the building of a transposed map, in one launch.  (1) mask[0] >= 4
// iff some cell holds more than two entries (bits [0, min(cnt, kTransSlots))), and row_mask
// says in which rows of the destination; with a second level, mask[1] holds the bits of the
// second-level slots in use (0: none).  (2) Clear
// the fp32 image the overflow list is accumulated into, only when the list is in use and
// not empty.
__global__ void after_transposed_map_kernel(const int *__restrict__ cnt, int64_t cells,
                                            int *__restrict__ mask, int two_level,
                                            float *__restrict__ img, int64_t total,
                                            const int *__restrict__ overflow,
                                            int *__restrict__ row_mask, int64_t plane, int row_px) {
  __shared__ unsigned block_mask;
  if (threadIdx.x == 0) block_mask = 0;
  __syncthreads();
  unsigned m = 0;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < cells;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int c = cnt[e];
    m |= (1u << min(c, 2 * kTransSlots)) - 1u;
    // row_mask[y] != 0 iff a cell of destination row y holds more than two entries (cells are
    // [tap][pixel], `plane` pixels in rows of row_px; every writer stores the same value)
    if (c > 2) row_mask[(e % plane) / row_px] = 1;
  }
  for (int d = 32; d > 0; d >>= 1) m |= __shfl_xor(m, d);
  if ((threadIdx.x & 63) == 0 && m) atomicOr(&block_mask, m);
  __syncthreads();
  report_pairs_beyond_two(mask, block_mask & ((1u << kTransSlots) - 1u));
  if (two_level && threadIdx.x == 0) {
    const unsigned m2 = block_mask >> kTransSlots;
    if (m2 && (m2 & ~(unsigned)__hip_atomic_load(mask + 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT)))
      atomicOr(mask + 1, (int)m2);
  }
  if (overflow[0] != 0 || overflow[1] <= 0) return;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    img[i] = 0.f;
}

// What the scatter form needs before it runs, in one launch (a launch costs about 4 us even
// when every workgroup leaves at once, as here on maps the gather form handles):
// dst[b,c,:] = bias[c] (or 0), and the weights repacked W[s][d][k] -> Wq[k][dc][s][16]: per
// (tap, 16-channel block) a contiguous [Spad x 16] slice; s padded to 64, d padded to 16, zeros
// in the padding.  Runs only when the gate agrees (see above).
template <typename TD>
__global__ void init_scatter_kernel(float *__restrict__ dst, const TD *__restrict__ bias, int C,
                                    int64_t plane, int64_t total, const TD *__restrict__ w,
                                    float *__restrict__ wq, int S, int K, int Spad, int dchunks,
                                    const int *__restrict__ gate, int run_if_zero) {
  if (gate && ((*gate == 0) != (run_if_zero != 0))) return;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = bias ? to_f32(bias[(i / plane) % C]) : 0.f;
  const int64_t packed = (int64_t)K * dchunks * Spad * kScDC;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < packed;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int dl = (int)(e % kScDC);
    const int sl = (int)((e / kScDC) % Spad);
    const int dc = (int)((e / ((int64_t)kScDC * Spad)) % dchunks);
    const int k = (int)(e / ((int64_t)kScDC * Spad * dchunks));
    const int d = dc * kScDC + dl;
    wq[e] = (sl < S && d < C) ? to_f32(w[((int64_t)sl * C + d) * K + k]) : 0.f;
  }
}

template <typename TD>
__global__ void convert_planes_kernel(const float *__restrict__ src, TD *__restrict__ dst,
                                      int64_t total, const int *__restrict__ gate,
                                      int run_if_zero) {
  if (gate && ((*gate == 0) != (run_if_zero != 0))) return;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = from_f32<TD>(src[i]);
}

// Gather part of a map plan: every (map location, tap) resolved once to four (element index of
// the sampled image as bits, weight) entries - the four bilinear corners, or up to four
// nearest points with the rest zero - in the layout the gather-product kernel reads with
// `packed_map` (the same as a transposed map's cells).
template <int NCORN>
__global__ void build_gather_plan_kernel(const float *__restrict__ map,
                                         const float *__restrict__ iw, float2 *__restrict__ gmap,
                                         int np, int weighted, int wrap, int SH, int SW, int K,
                                         int64_t total) {
  // (a wave takes 64 consecutive locations of one tap: its stores are 512-byte runs)
  const int64_t t0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t run = t0 / (64 * (int64_t)K), pixels = total / K;
  const int r = (int)(t0 - run * 64 * K);
  const int64_t n = run * 64 + (r & 63);
  const int k = r >> 6;
  if (n >= pixels) return;
  const int64_t e = n * K + k;  // (location, tap)
  float2 out[kTransSlotsConst];
#pragma unroll
  for (int i = 0; i < kTransSlotsConst; i++) out[i] = make_float2(0.f, 0.f);
  for (int sp = 0; sp < np; sp++) {
    const int64_t q = e * np + sp;
    PairTap<NCORN> t;
    resolve_pairs<NCORN, 1>(map[q * 2], map[q * 2 + 1], SH, SW, wrap != 0,
                            weighted ? iw[q] : 1.f, t);
#pragma unroll
    for (int i = 0; i < NCORN; i++)
      if (sp * NCORN + i < kTransSlotsConst)
        out[sp * NCORN + i] = make_float2(__builtin_bit_cast(float, t.off[i]), t.wt[i]);
  }
#pragma unroll
  for (int i = 0; i < kTransSlotsConst; i++)  // stored [tap][slot][location]
    gmap[((int64_t)k * kTransSlotsConst + i) * pixels + n] = out[i];
}

// A map has a gather part when a tap is at most four (offset, weight) pairs.
static_assert(kPlanSlots == kTransSlots, "a plan's gather part has the cells of a transposed map");
bool gather_plan_applies(int interp, int64_t P) {
  const int64_t np = P > 0 ? P : 1;
  return np * (canonical_interp(interp) == kInterpNearest ? 1 : 4) <= 4;
}

struct ScatterScratch {
  size_t wq, wpt, cnt, tmap, tmap2, acc32, ovf, stage, total;  // byte offsets
  bool two_level;  // a second four-slot level, applied by a second gather pass
  int64_t ovf_cap;  // entries of the overflow list (0: none)
  bool transposed_path;
};

// elem: bytes per data element; a non-fp32 destination needs an fp32 accumulation
// image for the atomic path.  MH x MW x K x P: the map (P = 0: unweighted).
ScatterScratch scatter_scratch(int64_t B, int64_t S, int64_t D, int64_t K, int64_t DH, int64_t DW,
                               size_t elem, int64_t MH, int64_t MW, int64_t P) {
  ScatterScratch sc;
  size_t off = 0;
  sc.wq = off;
  off += align256((size_t)(K * ((D + kScDC - 1) / kScDC) * round_up(S, kScSC) * kScDC) * 4);
  const int64_t cells = DH * DW * K;
  sc.transposed_path = cells * kTransSlots * 2 <= 0x7fffffffLL;
  // Single-row maps (mesh signals) point anywhere, and their cells fill unevenly: with K * P
  // contributions per vertex on average a four-slot cell overflows often, an eight-slot
  // one rarely.
  sc.two_level = sc.transposed_path && MH == 1;
  sc.tmap2 = 0;
  // One fp32 image: the scatter kernel's accumulation image of a non-fp32 destination
  // ([B][D][DN]) or the channel-last overflow image ([B][DN][D padded to 64]); never both.
  sc.acc32 = off;
  {
    const int64_t scatter_img = elem != 4 ? B * D * DH * DW : 0;
    const int64_t overflow_img = sc.transposed_path ? B * DH * DW * round_up(D, kOT) : 0;
    off += align256((size_t)std::max(scatter_img, overflow_img) * 4);
  }
  sc.wpt = sc.cnt = sc.tmap = off;
  if (sc.transposed_path) {
    sc.wpt = off;
    off += align256((size_t)(K * round_up(S, kGC) * round_up(D, kOT)) * 4);
    sc.cnt = off;  // counters, the overflow flag and list length; cleared with tmap
    off += align256((size_t)(cells + 8 + DH) * 4);  // (and a word per destination row)
    sc.tmap = off;  // [tap][slot][pixel] (source pixel index as bits, weight)
    off += align256((size_t)cells * kTransSlots * 2 * 4);
    sc.tmap2 = off;
    if (sc.two_level) off += align256((size_t)cells * kTransSlots * 2 * 4);
  }
  // Overflow list: room for half of the contributions a bilinear map can make.
  sc.ovf = sc.stage = off;
  sc.ovf_cap = 0;
  if (sc.transposed_path) {
    sc.ovf_cap = std::min<int64_t>(MH * MW * K * (P ? P : 1) * 2, 0x3fffffffLL);
    off += align256((size_t)sc.ovf_cap * sizeof(OverflowEntry));
  }
  // channel-last copy of a single-row source, channel-block copy of a bf16 one (see
  // launch_gather_product)
  sc.stage = off;
  if (sc.transposed_path && (MH == 1 || elem == 2))
    off += align256((size_t)(B * MH * MW * round_up(S, kGC)) * 4);
  sc.total = off;
  return sc;
}

// Counters, flags, slots and overflow list of the transposed map of `map`, into the scratch
// (or plan) region that starts at `cnt`.
int build_transposed_map(const ScatterScratch &sc, const float *map, const float *iw, int *cnt,
                         const ModeArgs &m, int64_t DH, int64_t DW, int64_t MH, int64_t MW,
                         int64_t K, hipStream_t s, bool cleared = false) {
  char *region = (char *)cnt - sc.cnt;
  float2 *tmap = (float2 *)(region + sc.tmap);
  float2 *tmap2 = sc.two_level ? (float2 *)(region + sc.tmap2) : nullptr;
  OverflowEntry *ovf = (OverflowEntry *)(region + sc.ovf);
  int *flag = cnt + DH * DW * K;
  // (`cleared`: an earlier kernel on the stream has zeroed the region up to the overflow list)
  if (!cleared)
    if (int rc = fill_f32((float *)cnt, (int64_t)((sc.ovf - sc.cnt) / 4), 0.f, s)) return rc;
  const int64_t pixels = MH * MW;
  const unsigned blocks = (unsigned)(((pixels + 63) / 64 * 64 * K + 255) / 256);
  if (m.mode == kInterpNearest)
    hipLaunchKernelGGL(build_transposed_map_kernel<1>, dim3(blocks), dim3(256), 0, s, map, iw, cnt,
                       tmap, tmap2, flag, ovf, (int)sc.ovf_cap, m.np, m.weighted, m.wrap, (int)DH,
                       (int)DW, (int)MW, (int)K, pixels);
  else
    hipLaunchKernelGGL(build_transposed_map_kernel<4>, dim3(blocks), dim3(256), 0, s, map, iw, cnt,
                       tmap, tmap2, flag, ovf, (int)sc.ovf_cap, m.np, m.weighted, m.wrap, (int)DH,
                       (int)DW, (int)MW, (int)K, pixels);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

}  // namespace

// ---- plan: the transposed map of one sample map, kept by the caller across calls ----------
// Layout: the scratch region [cnt, stage) of mfma_product_scatter (counters, eight flag words,
// a word per destination row, slots, second-level slots, overflow list); flag word 4 holds the pair mask of the map itself,
// for the weight gradient.  Depends on the map, its interpolation and the two image sizes only.
// (followed, for maps of at most four points per tap, by the gather part: MH * MW * K cells of
// four resolved entries)
size_t mfma_gather_plan_offset(int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,
                               int64_t P) {
  const ScatterScratch sc = scatter_scratch(1, 1, 1, K, DH, DW, 4, MH, MW, P);
  return sc.transposed_path ? align256(sc.stage - sc.cnt) : 0;
}

size_t mfma_scatter_plan_bytes(int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,
                               int64_t P) {
  const ScatterScratch sc = scatter_scratch(1, 1, 1, K, DH, DW, 4, MH, MW, P);
  if (!sc.transposed_path) return 0;
  size_t n = align256(sc.stage - sc.cnt);
  if (P <= kTransSlots && MH * MW * K * kTransSlots * 2 <= 0x7fffffffLL)
    n += align256((size_t)(MH * MW * K) * kTransSlots * sizeof(float2));
  return n;
}

int mfma_scatter_plan_build(const float *map, const float *iw, void *plan, int64_t DH, int64_t DW,
                            int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                            hipStream_t s) {
  const ScatterScratch sc = scatter_scratch(1, 1, 1, K, DH, DW, 4, MH, MW, P);
  if (!sc.transposed_path) return MCX_E_SHAPE;
  const ModeArgs m = mode_args(interp, P);
  int *cnt = (int *)plan;
  const int64_t cells = DH * DW * K;
  int *flag = cnt + cells;
  if (int rc = build_transposed_map(sc, map, iw, cnt, m, DH, DW, MH, MW, K, s)) return rc;
  hipLaunchKernelGGL(after_transposed_map_kernel,
                     dim3((unsigned)std::min<int64_t>((cells + 255) / 256, 4096)), dim3(256), 0, s,
                     cnt, cells, flag + 2, sc.two_level ? 1 : 0, (float *)nullptr, (int64_t)0,
                     flag, flag + 8, DH * DW, (int)DW);
  MCX_HIP_CHECK_LAUNCH();
  if (m.np * (m.mode == kInterpNearest ? 1 : 4) == 4)
    if (int rc = launch_pair_mask(map, iw, flag + 4, m, DH, DW, MH * MW * K, s, true)) return rc;
  if (gather_plan_applies(interp, P) && MH * MW * K * kTransSlots * 2 <= 0x7fffffffLL) {
    float2 *gmap = (float2 *)((char *)plan + mfma_gather_plan_offset(DH, DW, MH, MW, K, P));
    const int64_t total = MH * MW * K;
    const dim3 grid((unsigned)(((MH * MW + 63) / 64 * 64 * K + 255) / 256));
    if (m.mode == kInterpNearest)
      hipLaunchKernelGGL(build_gather_plan_kernel<1>, grid, dim3(256), 0, s, map, iw, gmap, m.np,
                         m.weighted, m.wrap, (int)DH, (int)DW, (int)K, total);
    else
      hipLaunchKernelGGL(build_gather_plan_kernel<4>, grid, dim3(256), 0, s, map, iw, gmap, m.np,
                         m.weighted, m.wrap, (int)DH, (int)DW, (int)K, total);
    MCX_HIP_CHECK_LAUNCH();
  }
  return 0;
}

size_t mfma_product_scatter_bytes(int64_t B, int64_t S, int64_t D, int64_t K, int64_t DH,
                                  int64_t DW, size_t elem, int64_t MH, int64_t MW, int64_t P) {
  return scatter_scratch(B, S, D, K, DH, DW, elem, MH, MW, P).total;
}

// dst is fully overwritten: dst[b,d] = bias[d] (or 0) + scattered products.
// scratch: mfma_product_scatter_bytes(...) bytes.
template <typename TD>
int mfma_product_scatter(const TD *src, const float *map, const float *iw, const TD *w,
                         const TD *bias, TD *dst, void *scratch, int64_t B, int64_t S, int64_t D,
                         int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                         int interp, hipStream_t s, const void *plan) {
  const ScatterScratch sc = scatter_scratch(B, S, D, K, DH, DW, sizeof(TD), MH, MW, P);
  char *base = (char *)scratch;
  // a plan is the transposed map of this very map, built earlier by mfma_scatter_plan_build:
  // the part of the scratch from the counters up to the staging area, ready to use
  char *pbase = plan ? (char *)const_cast<void *>(plan) - sc.cnt : base;
  float *wq = (float *)(base + sc.wq);
  const int Spad = (int)round_up(S, kScSC), dchunks = (int)((D + kScDC - 1) / kScDC);
  const ModeArgs m = mode_args(interp, P);
  const int *gate = nullptr;

  if (sc.transposed_path) {
    // build the transposed map, then try the atomic-free gather form first
    int *cnt = (int *)(pbase + sc.cnt);
    float2 *tmap = (float2 *)(pbase + sc.tmap);
    float2 *tmap2 = sc.two_level ? (float2 *)(pbase + sc.tmap2) : nullptr;
    float *wpt = (float *)(base + sc.wpt);
    const int64_t cells = DH * DW * K;
    int *flag = cnt + cells;
    gate = flag;
    OverflowEntry *ovf = (OverflowEntry *)(pbase + sc.ovf);
    TD *stage = (MH == 1 || sizeof(TD) == 2) ? (TD *)(base + sc.stage) : nullptr;
    // (the packing launch also clears the transposed map's counters, flags and slots)
    if (int rc = launch_pack_weights<TD>(
            w, wpt, D, S, K, 1, s, nullptr,
            plan ? ZeroJob{nullptr, 0}
                 : ZeroJob{reinterpret_cast<uint4 *>(cnt), (int64_t)((sc.ovf - sc.cnt) / 16)}))
      return rc;
    if (!plan)
      if (int rc = build_transposed_map(sc, map, iw, cnt, m, DH, DW, MH, MW, K, s, true))
        return rc;
    // What did not fit the four slots of its cell is accumulated with float atomics into a
    // channel-last fp32 image (cleared only when there is anything to add), which the
    // gather's epilogue adds.
    const int64_t Spad16 = round_up(S, kGC);
    const bool cl = stage != nullptr && use_channel_last(MH, kInterpNearest) &&
                    MH * MW * Spad16 * (int64_t)sizeof(TD) <= 0xffffffffLL;
    float *img = (float *)(base + sc.acc32);
    const int64_t total_img = B * DH * DW * round_up(D, kOT);
    // flag[2]: at least 4 iff some cell holds more than two entries (a plan has it already)
    hipLaunchKernelGGL(after_transposed_map_kernel,
                       dim3((unsigned)std::min<int64_t>(
                           std::max((total_img + 1023) / 1024, (cells + 255) / 256), 4096)),
                       dim3(256), 0, s, cnt, plan ? (int64_t)0 : cells, flag + 2,
                       sc.two_level ? 1 : 0, img, total_img, flag, flag + 8, DH * DW, (int)DW);
    MCX_HIP_CHECK_LAUNCH();
    if (cl) {  // the overflow pass reads the channel-last copy before the gather would make it
      dim3 tg((unsigned)((MH * MW + 63) / 64), (unsigned)((Spad16 + 63) / 64), (unsigned)B);
      hipLaunchKernelGGL(to_channel_last_kernel<TD>, tg, dim3(256), 0, s, src, stage, (int)S,
                         (int)Spad16, MH * MW);
      MCX_HIP_CHECK_LAUNCH();
    }
    hipLaunchKernelGGL(overflow_scatter_kernel<TD>, dim3(2048, (unsigned)B), dim3(64), 0, s, src,
                       cl ? (const TD *)stage : (const TD *)nullptr, (const void *)wpt, img, ovf,
                       flag, (int)sc.ovf_cap, (int)S, (int)Spad16, (int)D, (int)round_up(D, kOT),
                       MH * MW, DH * DW);
    MCX_HIP_CHECK_LAUNCH();
    if (int rc = launch_gather_product<TD>(src, (const float *)tmap, nullptr, wpt, bias, dst,
                                           stage, B, S, D, MH, MW, DH, DW, K, kTransSlots,
                                           kInterpNearest, gate, 1, s, img, cl, flag + 2, true,
                                           false, flag + 8))
      return rc;
    if (sc.two_level)  // entries five to eight of every cell, added onto dst
      if (int rc = launch_gather_product<TD>(src, (const float *)tmap2, nullptr, wpt,
                                             (const TD *)nullptr, dst, stage, B, S, D, MH, MW, DH,
                                             DW, K, kTransSlots, kInterpNearest, gate, 1, s,
                                             nullptr, cl, flag + 3, true, true))
        return rc;
  }

  // atomic path (runs when there is no transposed map or it overflowed)
  const int64_t total_dst = B * D * DH * DW;
  float *acc = sizeof(TD) == 4 ? (float *)dst : (float *)(base + sc.acc32);
  const unsigned fill_blocks = (unsigned)std::min<int64_t>((total_dst + 1023) / 1024, 8192);
  hipLaunchKernelGGL(init_scatter_kernel<TD>, dim3(fill_blocks), dim3(256), 0, s, acc, bias, (int)D,
                     DH * DW, total_dst, w, wq, (int)S, (int)K, Spad, dchunks, gate, 0);
  MCX_HIP_CHECK_LAUNCH();
  const int tiles_x = (int)((MW + kScPx - 1) / kScPx);
  const int64_t tiles_per_img = (int64_t)tiles_x * MH;
  const int64_t total = tiles_per_img * B;
  if (total > 0x7fffffffLL) return MCX_E_SHAPE;
  dim3 grid((unsigned)total);
#define MCX_LAUNCH(NCORN, NP)                                                                    \
  hipLaunchKernelGGL((product_scatter_mfma_kernel<TD, NCORN, NP>), grid, dim3(kScThreads), 0, s, \
                     src, map, iw, wq, acc, (int)S, (int)D, Spad, (int)DH, (int)DW, (int)MH,     \
                     (int)MW, (int)K, m.weighted, m.wrap, tiles_x, (int)tiles_per_img, gate, 0)
  MCX_DISPATCH_TAPS(m, MCX_LAUNCH)
#undef MCX_LAUNCH
  MCX_HIP_CHECK_LAUNCH();
  if (sizeof(TD) != 4) {
    hipLaunchKernelGGL(convert_planes_kernel<TD>, dim3(fill_blocks), dim3(256), 0, s, acc, dst,
                       total_dst, gate, 0);
    MCX_HIP_CHECK_LAUNCH();
  }
  return 0;
}

// ---- bias gradient for bf16 (fp32 accumulation) ---------------------------------------
namespace {
template <typename TD>
__global__ __launch_bounds__(256) void channel_sum_partial_td_kernel(const TD *__restrict__ g,
                                                                     float *__restrict__ part,
                                                                     int C, int N, int splits) {
  const int c = blockIdx.x, b = blockIdx.y, sp = blockIdx.z;
  const int per = (N + splits - 1) / splits;
  const int n0 = sp * per, n1 = min(N, n0 + per);
  const TD *p = g + ((int64_t)b * C + c) * N;
  float acc = 0.f;
  for (int n = n0 + threadIdx.x; n < n1; n += 256) acc += to_f32(p[n]);
  __shared__ float red[256];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride) red[threadIdx.x] += red[threadIdx.x + stride];
    __syncthreads();
  }
  if (threadIdx.x == 0) part[(int64_t)c * gridDim.y * splits + b * splits + sp] = red[0];
}
template <typename TD>
__global__ void channel_sum_final_td_kernel(const float *__restrict__ part, TD *__restrict__ gb,
                                            int C, int per_channel) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  float acc = 0.f;
  for (int i = 0; i < per_channel; i++) acc += part[(int64_t)c * per_channel + i];
  gb[c] = from_f32<TD>(acc);
}
inline int bias_splits(int64_t B, int64_t C, int64_t N) {
  int splits = 1;
  while (B * C * splits < 2048 && N / (splits * 2) >= 4096 && splits < 64) splits *= 2;
  return splits;
}
}  // namespace

size_t mfma_bias_grad_bytes(int64_t B, int64_t C, int64_t N) {
  return align256((size_t)(B * C * bias_splits(B, C, N)) * sizeof(float));
}

template <typename TD>
int mfma_bias_grad(const TD *g, TD *gb, void *scratch, int64_t B, int64_t C, int64_t N,
                   hipStream_t s) {
  const int splits = bias_splits(B, C, N);
  float *part = (float *)scratch;
  hipLaunchKernelGGL(channel_sum_partial_td_kernel<TD>, dim3((unsigned)C, (unsigned)B,
                                                             (unsigned)splits),
                     dim3(256), 0, s, g, part, (int)C, (int)N, splits);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(channel_sum_final_td_kernel<TD>, dim3((unsigned)((C + 63) / 64)), dim3(64), 0,
                     s, part, gb, (int)C, (int)(B * splits));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

#define MCX_INSTANTIATE_TD(TD)                                                                     \
  template int mfma_gather_product<TD>(const TD *, const float *, const float *, const TD *,      \
                                       const TD *, TD *, void *, int64_t, int64_t, int64_t,       \
                                       int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, \
                                       hipStream_t, const void *);                                \
  template int mfma_weight_grad<TD>(const TD *, const TD *, const float *, const float *, TD *,   \
                                    void *, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, \
                                    int64_t, int64_t, int64_t, int, hipStream_t, TD *,            \
                                    const void *);                                                \
  template int mfma_product_scatter<TD>(const TD *, const float *, const float *, const TD *,     \
                                        const TD *, TD *, void *, int64_t, int64_t, int64_t,      \
                                        int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,     \
                                        int, hipStream_t, const void *);                          \
  template int mfma_bias_grad<TD>(const TD *, TD *, void *, int64_t, int64_t, int64_t,            \
                                  hipStream_t);
MCX_INSTANTIATE_TD(float)
MCX_INSTANTIATE_TD(bf16_t)

}  // namespace mcx

namespace mcx {
void set_profile_events(void *start, void *stop) {
  g_prof_start = (hipEvent_t)start;
  g_prof_stop = (hipEvent_t)stop;
}
}  // namespace mcx
