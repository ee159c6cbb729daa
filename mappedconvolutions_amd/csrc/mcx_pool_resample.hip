// Bandwidth-bound map-driven gathers and scatters: resample_from_map /
// resample_to_map, mapped max / average pooling and their unpooling adjoints,
// plain and weighted.  One thread owns one map location and a chunk of CH
// channels: the tap (offsets + weights) is resolved once and applied to each of
// the thread's channel planes, so map decoding is amortised and neighbouring lanes
// read neighbouring pixels.  Pooling and unpooling have a second form, chosen per
// wave on the device: where the taps (or the transposed lists) of a wave's 64
// locations read a few short runs of the source, those runs are staged in LDS with
// 16-byte loads and the taps read LDS (window_pool, window_unpool).
#include <type_traits>

#include "mcx_device.h"
#include "mcx_plan.h"

namespace mcx {
namespace {

constexpr int kThreads = 256;
constexpr int kCH = 8;  // channels per thread
// Channels per thread of the pooling gather that keeps its taps in registers: resolving 9 taps
// costs about as much as sampling 6 channels, so it is spread over more of them.
constexpr int kPoolCH = 64;
// Map locations per workgroup: a 32 x 8 patch for resampling (arbitrary maps: neighbouring
// rows of the map read neighbouring source pixels), one 256-long row segment for pooling
// (taps already reach into the rows above and below; longer rows mean fewer cache lines
// per wave-wide load).
template <int OP>
struct Patch {
  static constexpr int kW = OP == 0 ? 32 : kThreads;
  static constexpr int kH = kThreads / kW;
};

enum { OP_RESAMPLE = 0, OP_AVG = 1, OP_MAX = 2 };

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Neighbouring rows
// of a map read the same source rows, so every XCD is given one contiguous run of the
// launch's work items: a row read again by the next row of outputs then hits in L2 instead
// of going to memory a second and third time.
__device__ inline int xcd_contiguous(int wg, int total) {
  const int q = total >> 3, r = total & 7;
  const int xcd = wg & 7, slot = wg >> 3;
  return xcd * q + min(xcd, r) + slot;
}

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
// The work of one thread: map location n, channels [c0, c0 + kCH) of image b.
template <typename T, int MODE, int OP>
__device__ inline void direct_gather(const T *__restrict__ in, const T *__restrict__ map,
                                     const T *__restrict__ iw, T *__restrict__ out,
                                     int64_t *__restrict__ idx, int C, int IH, int IW, int N,
                                     int K, int P, int n, int c0, int b, int cpt, bool ring) {
  // cpt: channels per thread, kPoolCH on the register-tap path below and kCH otherwise.
  // Every loop below is free of per-lane branches: loads are unconditional (see load_elem),
  // channels past the last one re-read the last plane (wave-uniform clamp) and are dropped
  // at the store, so that all loads of a step are in flight together.
  const int64_t plane = (int64_t)IH * IW;
  const unsigned plane_bytes = (unsigned)(plane * (int64_t)sizeof(T));
  const T *src = in + ((int64_t)b * C + c0) * plane;
  const int pm = P == 0 ? 1 : P;
  const int nc = min(cpt, C - c0);
  const int64_t o = ((int64_t)b * C + c0) * N + n;

  if constexpr (OP != OP_RESAMPLE) {
    // Pooling with few unweighted taps: resolve them all first and walk the channels in the
    // outer loop, so that the K x 2..4 reads of one channel's few source rows follow each
    // other closely and hit in cache (with the taps outside, a line was gone before the
    // next tap came back to it: every sampled byte came from memory).
    constexpr int kTaps = 9;
    if (P == 0) {
      // More than kTaps taps: groups of kTaps, each a pass over the planes that continues
      // from the value (and winner) the pass before left in the output, so the additions and
      // the comparisons keep the order of the taps.
      for (int k0 = 0; k0 < K; k0 += kTaps) {
        const int kn = min(kTaps, K - k0);
        const bool first = k0 == 0, last = k0 + kTaps >= K;
        Tap<T, MODE> taps[kTaps];
#pragma unroll
        for (int k = 0; k < kTaps; k++) {
          const int64_t e = (int64_t)n * K + min(k0 + k, K - 1);
          taps[k].set(map[e * 2], map[e * 2 + 1], IH, IW);
        }
        // wave-uniform: bit k set when some lane uses row 0 / row 1 of tap k, and when every
        // lane's tap k can fetch a row's two corners with one load
        unsigned rows0 = 0, rows1 = 0, pairs = 0;
#pragma unroll
        for (int k = 0; k < kTaps; k++) {
          rows0 |= __builtin_amdgcn_ballot_w64(taps[k].row_in_use(0)) ? 1u << k : 0u;
          rows1 |= __builtin_amdgcn_ballot_w64(taps[k].row_in_use(1)) ? 1u << k : 0u;
          pairs |= __builtin_amdgcn_ballot_w64(!taps[k].pairable()) ? 0u : 1u << k;
        }
        for (int c = 0; c < nc; c++) {
          const plane_buf_t pl = plane_buf(src + c * plane, plane_bytes);
          // every load of the channel is issued before the first one is used (left to itself
          // the compiler interleaves loads and waits to save registers, one load in flight)
          T a = OP == OP_MAX ? T(-3.402823466e+38F) : T(0);
          int64_t best = -1;
          if (!first) {  // (uniform over the launch)
            a = out[o + (int64_t)c * N];
            if (OP == OP_MAX) best = idx[o + (int64_t)c * N];
          }
          T d[kTaps][Tap<T, MODE>::kCorners];
#pragma unroll
          for (int k = 0; k < kTaps; k++)
            taps[k].load_rows(pl, d[k], (rows0 >> k) & 1u, (rows1 >> k) & 1u, (pairs >> k) & 1u);
          __builtin_amdgcn_sched_barrier(0);
          T val[kTaps];
#pragma unroll
          for (int k = 0; k < kTaps; k++) val[k] = taps[k].combine(d[k]);
          int bk = -1;
#pragma unroll
          for (int k = 0; k < kTaps; k++) {
            if (OP == OP_MAX) {
              const bool better = k < kn && val[k] > a;
              a = better ? val[k] : a;
              bk = better ? k : bk;
            } else {
              a = k < kn ? a + val[k] : a;
            }
          }
          out[o + (int64_t)c * N] = (OP == OP_AVG && last) ? a / (T)K : a;
          if (OP == OP_MAX)
            idx[o + (int64_t)c * N] = bk < 0 ? best : ((int64_t)n * K + k0 + bk) * 2;
        }
      }
      return;
    }
  }
  if constexpr (OP == OP_RESAMPLE) {
    // Resampling without interpolation weights (one tap per location): the tap is resolved
    // once and the planes are walked with the loads of kRing of them in flight; a plane's
    // value is stored when its loads have arrived and its registers take the loads of the
    // plane kRing further on.  Loads and stores are unconditional (planes past the last one
    // re-read the last plane and store out of range), so the waits count exactly.
    if (ring) {
      constexpr int kRing = 8, kCorners = Tap<T, MODE>::kCorners;
      Tap<T, MODE> tap;
      tap.set(map[(int64_t)n * 2], map[(int64_t)n * 2 + 1], IH, IW);
      const unsigned n_bytes = (unsigned)N * (unsigned)sizeof(T);
      const unsigned o_off = (unsigned)n * (unsigned)sizeof(T);
      T *dst = out + ((int64_t)b * C + c0) * N;
      auto run = [&](auto pairs_tag) {
        constexpr bool PAIRS = decltype(pairs_tag)::value;
        T d[kRing][kCorners];
#pragma unroll
        for (int u = 0; u < kRing; u++)
          tap.template load_flat<PAIRS>(plane_buf(src + min(u, nc - 1) * plane, plane_bytes), d[u]);
        int cb = 0;
        for (; cb + kRing < nc; cb += kRing) {
#pragma unroll
          for (int u = 0; u < kRing; u++) {
            const int c = cb + u;
            buf_store(plane_buf(dst + (int64_t)c * N, n_bytes), o_off, tap.combine(d[u]));
            tap.template load_flat<PAIRS>(
                plane_buf(src + min(c + kRing, nc - 1) * plane, plane_bytes), d[u]);
          }
        }
#pragma unroll
        for (int u = 0; u < kRing; u++) {  // the last ring: nothing left to load
          const int c = cb + u;
          buf_store(plane_buf(dst + (int64_t)min(c, nc - 1) * N, n_bytes),
                    c < nc ? o_off : kOobOffset, tap.combine(d[u]));
        }
      };
      if (kCorners == 4 && __builtin_amdgcn_ballot_w64(!tap.pairable()) == 0)
        run(std::true_type());
      else
        run(std::false_type());
      return;
    }
  }
  plane_buf_t pl[kCH];
#pragma unroll
  for (int c = 0; c < kCH; c++) pl[c] = plane_buf(src + min(c, nc - 1) * plane, plane_bytes);
  T acc[kCH];
  int64_t best[kCH];
#pragma unroll
  for (int c = 0; c < kCH; c++) {
    acc[c] = OP == OP_MAX ? T(-3.402823466e+38F) : T(0);
    best[c] = -1;
  }
  // Unweighted: the next tap's coordinates are fetched while this tap's samples are.
  T nx = T(0), ny = T(0);
  if (P == 0) {
    nx = map[(int64_t)n * K * 2];
    ny = map[(int64_t)n * K * 2 + 1];
  }
  for (int k = 0; k < K; k++) {
    const int64_t e = ((int64_t)n * K + k) * pm;
    T val[kCH];
    if (P == 0) {
      Tap<T, MODE> tap;
      tap.set(nx, ny, IH, IW);
      if (k + 1 < K) {
        nx = map[(e + 1) * 2];
        ny = map[(e + 1) * 2 + 1];
      }
      const bool row0 = __builtin_amdgcn_ballot_w64(tap.row_in_use(0)) != 0;
      const bool row1 = __builtin_amdgcn_ballot_w64(tap.row_in_use(1)) != 0;
      const bool pairs = __builtin_amdgcn_ballot_w64(!tap.pairable()) == 0;
      T d[kCH][Tap<T, MODE>::kCorners];
#pragma unroll
      for (int c = 0; c < kCH; c++) tap.load_rows(pl[c], d[c], row0, row1, pairs);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < kCH; c++) val[c] = tap.combine(d[c]);
    } else {
#pragma unroll
      for (int c = 0; c < kCH; c++) val[c] = T(0);
      for (int p = 0; p < P; p++) {
        Tap<T, MODE> tap;
        tap.set(map[(e + p) * 2], map[(e + p) * 2 + 1], IH, IW);
        const T w = iw[e + p];
        const bool row0 = __builtin_amdgcn_ballot_w64(tap.row_in_use(0)) != 0;
        const bool row1 = __builtin_amdgcn_ballot_w64(tap.row_in_use(1)) != 0;
        const bool pairs = __builtin_amdgcn_ballot_w64(!tap.pairable()) == 0;
        T d[kCH][Tap<T, MODE>::kCorners];
#pragma unroll
        for (int c = 0; c < kCH; c++) tap.load_rows(pl[c], d[c], row0, row1, pairs);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < kCH; c++) val[c] += w * tap.combine(d[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < kCH; c++) {
      if (OP == OP_MAX) {
        const bool better = val[c] > acc[c];
        acc[c] = better ? val[c] : acc[c];
        best[c] = better ? e * 2 : best[c];
      } else if (OP == OP_AVG) {
        acc[c] += val[c];
      } else {
        acc[c] = val[c];
      }
    }
  }
#pragma unroll
  for (int c = 0; c < kCH; c++) {
    if (c >= nc) continue;
    out[o + (int64_t)c * N] = OP == OP_AVG ? acc[c] / (T)K : acc[c];
    if (OP == OP_MAX) idx[o + (int64_t)c * N] = best[c];
  }
}

// ---------------------------------------------------------------------------------
// Pooling through LDS windows.  The texture path resolves four lanes' addresses per clock
// whatever the width of the load, so a gather of single elements (nine taps of two corners
// per output and channel) is bound by it long before memory.  Where the taps of a wave's 64
// neighbouring outputs read a few source rows over short spans - the distortion-aware kernels
// of equirectangular images do: every tap of a row segment stays in one source row and moves
// with the pixel - those spans are copied to LDS with 16-byte loads, one lane per four
// elements, and the taps read LDS.  Every wave works alone (its own windows, no workgroup
// barrier) and finds its spans from the map itself:
//   * per (tap, corner row): the source row must be the same for every lane that uses it,
//     and the columns must lie within a short distance (cyclic in the width, so a seam
//     inside the segment is no obstacle) after the first lane's;
//   * entries of one source row that lie close together share a row window; lane s of the
//     wave keeps row window s while they are merged;
//   * if anything does not fit, the wave takes the register path above.
// The arithmetic per output is that of the register path (Tap::combine on the same values).
// ---------------------------------------------------------------------------------
constexpr int kWinChunks = 128;   // 16-byte chunks per window, followed by one of zeros
constexpr int kWinRows = 6;
constexpr int kWinSpanCap = 400;  // elements between the first and the last column of a span
constexpr int kWinTaps = 9;
constexpr int kWinDepth = 4;      // channels whose loads are in flight

template <typename T, int MODE>
struct WinShape {
  static constexpr int kRowsPerTap = Tap<T, MODE>::kCorners == 4 ? 2 : 1;
  static constexpr int kColsPerRow = Tap<T, MODE>::kCorners == 4 ? 2 : 1;
  static constexpr int kEntries = kWinTaps * kRowsPerTap;
};

__device__ inline int cyc(int v, int w) { return v < 0 ? v + w : v; }  // v in (-w, w)

// Largest value of the wave (all 64 lanes active), by data-parallel-primitive moves inside the
// vector unit: shifts within rows of 16 lanes, then the rows' last lanes passed on; lanes a
// step does not reach keep the identity.  (Shuffles go through LDS, a round trip per step.)
__device__ inline int wave_max(int v) {
  constexpr int kId = -0x7fffffff - 1;
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x111, 0xf, 0xf, false));  // row_shr:1
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x112, 0xf, 0xf, false));  // row_shr:2
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x114, 0xf, 0xe, false));  // row_shr:4
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x118, 0xf, 0xc, false));  // row_shr:8
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x142, 0xa, 0xf, false));  // row_bcast:15
  v = max(v, __builtin_amdgcn_update_dpp(kId, v, 0x143, 0xc, 0xf, false));  // row_bcast:31
  return __builtin_amdgcn_readlane(v, 63);
}

// Returns false (wave-uniform) when the wave's taps do not fit windows; nothing is written then.
template <typename T, int MODE, int OP>
__device__ inline bool window_pool(const T *__restrict__ in, const T *__restrict__ map,
                                   T *__restrict__ out, int64_t *__restrict__ idx, int C, int IH,
                                   int IW, int N, int K, int n, bool live, int c0, int b,
                                   int cpt) {
  using Shape = WinShape<T, MODE>;
  constexpr int kRPT = Shape::kRowsPerTap, kCPR = Shape::kColsPerRow, kEnt = Shape::kEntries;
  constexpr int kCorners = Tap<T, MODE>::kCorners;
  constexpr int kPer = 16 / (int)sizeof(T);  // elements per chunk
  constexpr unsigned kZeroOff = kWinChunks * 16;
  __shared__ uint4 win[kThreads / 64][2][kWinChunks + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // this thread's taps, and for every tap the row / (cyclic) column of its first corner
  Tap<T, MODE> taps[kWinTaps];
  int ty[kWinTaps], tx[kWinTaps];
#pragma unroll
  for (int k = 0; k < kWinTaps; k++) {
    const int64_t e = (int64_t)(live ? n : 0) * K + min(k, K - 1);
    const T x = map[e * 2], y = map[e * 2 + 1];
    taps[k].set(x, y, IH, IW);
    if (MODE == kInterpNearest) {
      tx[k] = to_int(round_half_away(x));
      ty[k] = to_int(round_half_away(y));
    } else {
      tx[k] = to_int(mcx_floor(x));
      ty[k] = to_int(mcx_floor(y));
    }
    tx[k] = wrap_index(tx[k], IW);
  }
  // Entries: (tap, corner row) pairs in use.  Everything about them is wave-uniform.
  bool fits = true;
  unsigned rows_used = 0;  // bit (k * kRPT + r)
  int e_row[kEnt], e_col[kEnt], e_len[kEnt];
#pragma unroll
  for (int k = 0; k < kWinTaps; k++) {
#pragma unroll
    for (int r = 0; r < kRPT; r++) {
      const int e = k * kRPT + r;
      const bool use = live && k < K && taps[k].row_in_use(r);
      const unsigned long long bu = __builtin_amdgcn_ballot_w64(use);
      e_row[e] = e_col[e] = e_len[e] = 0;
      if (bu) {
        const int first = __builtin_ctzll(bu);
        const int row = ty[k] + r;
        e_row[e] = __builtin_amdgcn_readlane(row, first);
        e_col[e] = __builtin_amdgcn_readlane(tx[k], first);
        const int far = wave_max(use ? cyc(tx[k] - e_col[e], IW) : 0);
        if (__builtin_amdgcn_ballot_w64(use && row != e_row[e]) != 0 || far > kWinSpanCap)
          fits = false;
        e_len[e] = far + kCPR;
        rows_used |= 1u << e;
      }
    }
  }
  // Second corner rows in use (row coordinates that are not integral): four offsets and
  // weights per tap plus the loads in flight do not fit the register budget of four waves per
  // SIMD, and spilling inside the channel loop costs more than the texture path does.
  constexpr unsigned kSecondRows = kRPT == 2 ? 0x2aaaau : 0u;  // bits k * 2 + 1
  if (!fits || !rows_used || (rows_used & kSecondRows)) return false;
  // Row windows: lane s keeps window s (source row, first column, length in elements).
  int r_row = 0, r_start = 0, r_len = 0, nrows = 0;
  int e_slot[kEnt];
#pragma unroll
  for (int e = 0; e < kEnt; e++) {
    e_slot[e] = 0;
    if ((rows_used >> e) & 1u) {
      const int d = cyc(e_col[e] - r_start, IW), d2 = cyc(r_start - e_col[e], IW);
      const bool mine = lane < nrows && r_row == e_row[e] && min(d, d2) <= kWinSpanCap;
      const unsigned long long bm = __builtin_amdgcn_ballot_w64(mine);
      if (bm) {
        e_slot[e] = __builtin_ctzll(bm);
        if (lane == e_slot[e]) {
          if (d <= d2) {  // starts inside or after the window
            r_len = max(r_len, d + e_len[e]);
          } else {  // starts before it
            r_len = max(e_len[e], d2 + r_len);
            r_start = e_col[e];
          }
        }
      } else {
        e_slot[e] = nrows;
        if (lane == nrows) {
          r_row = e_row[e];
          r_start = e_col[e];
          r_len = e_len[e];
        }
        nrows++;
      }
    }
  }
  // windows start on a chunk boundary; one that reaches all the way round is the whole row
  int r_first = r_start & ~(kPer - 1);
  r_len += r_start - r_first;
  if (r_len >= IW) {
    r_len = IW;
    r_first = 0;
  }
  const int r_chunks = lane < nrows ? (r_len + kPer - 1) / kPer : 0;
  int r_chunk0 = 0, chunks = 0;
#pragma unroll
  for (int s2 = 0; s2 < kWinRows; s2++) {
    if (lane == s2) r_chunk0 = chunks;
    chunks += __builtin_amdgcn_readlane(r_chunks, s2);
  }
  if (nrows > kWinRows || chunks > kWinChunks) return false;

  // LDS byte offset of every corner (the zero chunk for corners outside the plane or of
  // weight zero), kept where the register path keeps the element offsets
#pragma unroll
  for (int k = 0; k < kWinTaps; k++) {
#pragma unroll
    for (int r = 0; r < kRPT; r++) {
      const int e = k * kRPT + r;
      const bool used = (rows_used >> e) & 1u;
      const int first = __builtin_amdgcn_readlane(r_first, e_slot[e]);
      const int base = __builtin_amdgcn_readlane(r_chunk0, e_slot[e]) * kPer;
      const int col = cyc(tx[k] - first, IW);
#pragma unroll
      for (int i = 0; i < kCPR; i++) {
        int cc = col + i;
        cc = cc >= IW ? cc - IW : cc;
        const bool valid = live && used && taps[k].corner_off(r * kCPR + i) >= 0;
        taps[k].set_corner_off(r * kCPR + i,
                               valid ? (int)((unsigned)(base + cc) * (unsigned)sizeof(T))
                                     : (int)kZeroOff);
      }
    }
  }
  // the chunks this lane copies per channel: byte offset in the plane, or out of range
  unsigned goff[2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int q = lane + j * 64;
    goff[j] = kOobOffset;
#pragma unroll
    for (int s2 = 0; s2 < kWinRows; s2++) {
      const int c_0 = __builtin_amdgcn_readlane(r_chunk0, s2);
      const int c_n = __builtin_amdgcn_readlane(r_chunks, s2);
      const int c_y = __builtin_amdgcn_readlane(r_row, s2);
      const int c_x = __builtin_amdgcn_readlane(r_first, s2);
      int x = c_x + (q - c_0) * kPer;
      x = x >= IW ? x - IW : x;
      if (q >= c_0 && q < c_0 + c_n) goff[j] = (unsigned)(c_y * IW + x) * (unsigned)sizeof(T);
    }
  }

  const int64_t plane = (int64_t)IH * IW;
  const unsigned plane_bytes = (unsigned)(plane * (int64_t)sizeof(T));
  const T *src = in + ((int64_t)b * C + c0) * plane;
  const int nc = min(cpt, C - c0);
  const int64_t o_plane = ((int64_t)b * C + c0) * N;
  const int64_t idx_base = (int64_t)n * K * 2;
  // Per channel: its window's chunks travel memory -> registers -> LDS.  The loads of
  // kWinDepth channels are in flight (one channel's arithmetic is far shorter than a load's
  // latency); LDS holds two windows, the one being read and the one being filled.  A wave's
  // LDS accesses execute in order, so the wave needs no barrier between filling a window
  // and reading it; wave_barrier() only keeps the compiler from moving them.
  uint4 pre[kWinDepth][2];
  auto fetch = [&](int c, int slot) {
    const plane_buf_t pl = plane_buf(src + c * plane, plane_bytes);
#pragma unroll
    for (int j = 0; j < 2; j++)
      pre[slot][j] =
          __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(pl, (int)goff[j], 0, 0));
  };
  auto stash = [&](int slot, int buf) {
    win[wave][buf][lane] = pre[slot][0];
    win[wave][buf][lane + 64] = pre[slot][1];
    __builtin_amdgcn_wave_barrier();
  };
  if (lane < 2) win[wave][lane][kWinChunks] = make_uint4(0u, 0u, 0u, 0u);
  // FULL (all kWinTaps taps exist) is settled once per wave rather than per tap and channel,
  // with one copy of the channel loop for each answer.  Only the first corner row of a tap is
  // read: the products of the second are zeros here, so the sum differs from the register
  // path's at most in the sign of a zero.
  auto run = [&](auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    constexpr int kRead = kCPR;
    auto compute = [&](int c, int buf) {
      const char *wb = reinterpret_cast<const char *>(&win[wave][buf][0]);
      // every read is unconditional (a corner that is not in use reads the zero chunk), so
      // all of a channel's reads are in flight together
      T d[kWinTaps][kCorners];
#pragma unroll
      for (int k = 0; k < kWinTaps; k++)
#pragma unroll
        for (int i = 0; i < kRead; i++)
          d[k][i] = *reinterpret_cast<const T *>(wb + (unsigned)taps[k].corner_off(i));
      __builtin_amdgcn_sched_barrier(0);
      T val[kWinTaps];
#pragma unroll
      for (int k = 0; k < kWinTaps; k++) {
        if (kRead == kCorners)
          val[k] = taps[k].combine(d[k]);
        else
          val[k] = taps[k].corner_wt(0) * d[k][0] + taps[k].corner_wt(1) * d[k][1];
      }
      T a = OP == OP_MAX ? T(-3.402823466e+38F) : T(0);
      int bk = -1;
#pragma unroll
      for (int k = 0; k < kWinTaps; k++) {
        if (OP == OP_MAX) {
          const bool better = (FULL || k < K) && val[k] > a;
          a = better ? val[k] : a;
          bk = better ? k : bk;
        } else {
          a = (FULL || k < K) ? a + val[k] : a;
        }
      }
      // (stores without a branch: lanes past the row's end and channels past the last one
      // store out of range, which drops the store)
      const int cc = min(c, nc - 1);
      const bool keep = live && c < nc;
      buf_store(plane_buf(out + o_plane + (int64_t)cc * N, (unsigned)N * (unsigned)sizeof(T)),
                keep ? (unsigned)n * (unsigned)sizeof(T) : kOobOffset,
                OP == OP_AVG ? a / (T)K : a);
      if (OP == OP_MAX)
        buf_store(plane_buf(idx + o_plane + (int64_t)cc * N, (unsigned)N * 8u),
                  keep ? (unsigned)n * 8u : kOobOffset,
                  bk < 0 ? (int64_t)-1 : idx_base + 2 * bk);
      __builtin_amdgcn_wave_barrier();
    };
    // (the loop runs over a whole number of rings and re-reads the last channel past the end:
    // with the same loads and stores on every path the compiler can count how many may still
    // be in flight at each wait; a load behind a test makes every wait a full one)
#pragma unroll
    for (int u = 0; u < kWinDepth; u++) fetch(min(u, nc - 1), u);
    stash(0, 0);
    for (int cb = 0; cb < nc; cb += kWinDepth) {
#pragma unroll
      for (int u = 0; u < kWinDepth; u++) {
        const int c = cb + u;
        fetch(min(c + kWinDepth, nc - 1), u);  // slot u went to LDS in the previous step
        compute(c, u & 1);
        stash((u + 1) % kWinDepth, (u + 1) & 1);
      }
    }
  };
  if (K == kWinTaps)
    run(std::true_type());
  else
    run(std::false_type());
  return true;
}

template <typename T, int MODE, int OP>
__global__ __launch_bounds__(kThreads, 4) void gather_kernel(
    const T *__restrict__ in, const T *__restrict__ map, const T *__restrict__ iw,
    T *__restrict__ out, int64_t *__restrict__ idx, int C, int IH, int IW, int N, int MW, int K,
    int P, int cpt, int windows) {
  constexpr int kTileW = Patch<OP>::kW, kTileH = Patch<OP>::kH;
  const int tiles_x = (MW + kTileW - 1) / kTileW;
  // (pooling only: a resampling map's rows need not read neighbouring source rows, and the
  // round-robin order measured faster there)
  const int tile = OP == OP_RESAMPLE ? (int)blockIdx.x : xcd_contiguous(blockIdx.x, gridDim.x);
  const int tx = (tile % tiles_x) * kTileW + threadIdx.x % kTileW;
  const int ty = (tile / tiles_x) * kTileH + threadIdx.x / kTileW;
  const int n = ty * MW + tx;
  const bool live = tx < MW && n < N;
  if constexpr (OP != OP_RESAMPLE) {
    // `windows`: unweighted, at most kWinTaps taps, rows a whole number of 16-byte chunks
    if (windows && window_pool<T, MODE, OP>(in, map, out, idx, C, IH, IW, N, K, n, live,
                                            blockIdx.y * cpt, blockIdx.z, cpt))
      return;
  }
  if (!live) return;
  // (`windows` of a resampling launch: the plane ring of direct_gather applies)
  direct_gather<T, MODE, OP>(in, map, iw, out, idx, C, IH, IW, N, K, P, n, blockIdx.y * cpt,
                             blockIdx.z, cpt, OP == OP_RESAMPLE && windows != 0);
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


// ---- scatter ops as gathers through a transposed map -------------------------
// resample_to_map and the two unpoolings push every source value to the
// destination pixels its taps touch.  The map is shared by all B*C planes, so it
// pays to turn it around once per call: a compressed list, per destination pixel,
// of the (source location, weight) pairs that land on it (count -> prefix sum ->
// fill), after which every destination element is a plain weighted gather: no
// float atomics, no zero fill, each output written once.  Contributions whose
// weight is exactly zero are left out (they add 0 to any finite value).
constexpr int kScanItems = 8;                      // counts per thread of the block scan
constexpr int kScanBlock = kThreads * kScanItems;  // counts per block

enum { UN_RESAMPLE = 0, UN_AVG = 1, UN_MAX = 2 };

// One thread per source location n, walking its per_loc = K*Pm samples i = n*per_loc + q (with
// one thread per sample, the lanes of a wave - neighbouring taps of one location - hit
// destination pixels rows apart; with one thread per location they hit neighbouring pixels at
// every step, and the counters of a cache line are updated by one request: counting the
// 512 x 1024 x 9 pooling map took 0.087 ms with one thread per sample, 0.035 ms so; launched
// with per_loc = 1 the kernel is the one-thread-per-sample form).  FILL == false counts the
// contributions of each destination pixel; FILL == true writes them to their place.
template <typename T, int MODE, bool FILL>
__global__ __launch_bounds__(kThreads) void transposed_map_kernel(
    const T *__restrict__ map, const T *__restrict__ iw, int64_t nloc, int per_loc, int per_code,
    int DH, int DW, uint32_t *__restrict__ local, uint32_t *__restrict__ cursor,
    const uint32_t *__restrict__ bsum, uint32_t *__restrict__ e_src, T *__restrict__ e_wt) {
  const int64_t n = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (n >= nloc) return;
  for (int q = 0; q < per_loc; q++) {
    const int64_t i = n * per_loc + q;
    Tap<T, MODE> tap;
    tap.set(map[i * 2], map[i * 2 + 1], DH, DW);
    const T w = iw ? iw[i] : T(1);
    const uint32_t code = (uint32_t)(i / per_code);
#pragma unroll
    for (int c = 0; c < Tap<T, MODE>::kCorners; c++) {
      const int off = tap.corner_off(c);
      const T ww = iw ? tap.corner_wt(c) * w : tap.corner_wt(c);
      if (off < 0 || ww == T(0)) continue;
      if (!FILL) {
        atomicAdd(&local[off], 1u);
      } else {
        const uint32_t pos = local[off] + bsum[off / kScanBlock] + atomicAdd(&cursor[off], 1u);
        e_src[pos] = code;
        e_wt[pos] = ww;
      }
    }
  }
}

// Exclusive prefix sum of counts, two levels: within blocks of kScanBlock (in
// place), then over the block totals (one workgroup).  The prefix of element i is
// local[i] + bsum[i / kScanBlock].
__global__ __launch_bounds__(kThreads) void scan_blocks_kernel(uint32_t *__restrict__ local,
                                                               uint32_t *__restrict__ bsum,
                                                               int64_t n) {
  __shared__ uint32_t part[kThreads];
  const int64_t base = (int64_t)blockIdx.x * kScanBlock + (int64_t)threadIdx.x * kScanItems;
  uint32_t v[kScanItems], sum = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; j++) {
    v[j] = base + j < n ? local[base + j] : 0u;
    sum += v[j];
  }
  part[threadIdx.x] = sum;
  __syncthreads();
  for (int d = 1; d < kThreads; d <<= 1) {
    const uint32_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0u;
    __syncthreads();
    part[threadIdx.x] += add;
    __syncthreads();
  }
  uint32_t run = part[threadIdx.x] - sum;  // exclusive prefix of this thread
#pragma unroll
  for (int j = 0; j < kScanItems; j++) {
    if (base + j < n) local[base + j] = run;
    run += v[j];
  }
  if (threadIdx.x == kThreads - 1) bsum[blockIdx.x] = part[threadIdx.x];
}

__global__ __launch_bounds__(kThreads) void scan_sums_kernel(uint32_t *__restrict__ bsum, int n) {
  __shared__ uint32_t part[kThreads];
  uint32_t carry = 0;
  for (int base = 0; base < n; base += kThreads) {
    const int i = base + (int)threadIdx.x;
    const uint32_t v = i < n ? bsum[i] : 0u;
    part[threadIdx.x] = v;
    __syncthreads();
    for (int d = 1; d < kThreads; d <<= 1) {
      const uint32_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0u;
      __syncthreads();
      part[threadIdx.x] += add;
      __syncthreads();
    }
    if (i < n) bsum[i] = carry + part[threadIdx.x] - v;
    carry += part[kThreads - 1];
    __syncthreads();
  }
}

// Orders the entries of every destination pixel by source location (insertion sort,
// one thread per pixel; lists are short).  The fill kernel places entries in the
// order its atomics happen to retire: sorted lists make the result independent of
// that order, and neighbouring lanes of the gather then read neighbouring sources
// at the same step.  Lists longer than kSortMax stay as filled.
constexpr uint32_t kSortMax = 512;

// Batcher's odd-even merge sort for N keys (16 or 32) as a list of compare-exchange pairs, made
// at compile time so that the unrolled network indexes registers statically.
constexpr int kNetN = 32;
struct SortNetwork {
  int n;
  unsigned char a[256], b[256];
};
constexpr SortNetwork make_network(int N) {
  SortNetwork net{};
  for (int p = 1; p < N; p *= 2)
    for (int k = p; k >= 1; k /= 2)
      for (int j = k % p; j + k < N; j += 2 * k)
        for (int i = 0; i < k && i + j + k < N; i++)
          if ((i + j) / (2 * p) == (i + j + k) / (2 * p)) {
            net.a[net.n] = (unsigned char)(i + j);
            net.b[net.n] = (unsigned char)(i + j + k);
            net.n++;
          }
  return net;
}
constexpr SortNetwork kNet32 = make_network(32), kNet16 = make_network(16);

// Sorts the list [start, end) of this lane (at most N entries) in registers: read once, run
// through the network, written back.  Order: by source, ties by weight.
template <typename T, int N>
__device__ inline void network_sort(uint32_t *e_src, T *e_wt, uint32_t start, uint32_t end) {
  constexpr const SortNetwork &net = N == 16 ? kNet16 : kNet32;
  uint32_t code[N];
  T w[N];
#pragma unroll
  for (int u = 0; u < N; u++) {
    const bool in = start + u < end;
    code[u] = in ? e_src[start + u] : 0xffffffffu;  // padding sorts to the end
    w[u] = in ? e_wt[start + u] : T(0);
  }
#pragma unroll
  for (int c = 0; c < net.n; c++) {
    const int ia = net.a[c], ib = net.b[c];
    const bool swap = code[ia] > code[ib] || (code[ia] == code[ib] && w[ia] > w[ib]);
    const uint32_t ca = swap ? code[ib] : code[ia], cb = swap ? code[ia] : code[ib];
    const T wa = swap ? w[ib] : w[ia], wb = swap ? w[ia] : w[ib];
    code[ia] = ca; code[ib] = cb;
    w[ia] = wa; w[ib] = wb;
  }
#pragma unroll
  for (int u = 0; u < N; u++) {
    if (start + u < end) {
      e_src[start + u] = code[u];
      e_wt[start + u] = w[u];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void sort_entries_kernel(
    const uint32_t *__restrict__ local, const uint32_t *__restrict__ bsum,
    uint32_t *__restrict__ e_src, T *__restrict__ e_wt, int ndst) {
  const int p = blockIdx.x * kThreads + threadIdx.x;
  const bool live = p < ndst;
  const uint32_t start = live ? local[p] + bsum[p / kScanBlock] : 0u;
  const uint32_t end = live ? local[p + 1] + bsum[(p + 1) / kScanBlock] : 0u;
  // Lists of up to kNetN entries in every lane of the wave (pooling and resampling maps):
  // read once into registers, sorted by the network, written back.  Same order as the
  // insertion sort below: by source, ties by weight.
  // (a wave most of whose lists are very short is quicker with the insertion sort)
  if (__builtin_amdgcn_ballot_w64(end - start > (uint32_t)kNetN) == 0 &&
      __builtin_popcountll(__builtin_amdgcn_ballot_w64(end - start > 8u)) >= 32) {
    if (__builtin_amdgcn_ballot_w64(end - start > 16u) == 0) {
      // The lists of a wave's 64 pixels are one contiguous run of at most 1024 entries: it
      // is copied to LDS and back with coalesced accesses, and each lane sorts its piece
      // there (a lane's own list starts 15 or so words after its neighbour's: separate
      // cache lines in memory, separate banks in LDS).
      __shared__ uint32_t run_src[kThreads / 64][64 * 16];
      __shared__ T run_wt[kThreads / 64][64 * 16];
      const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
      const uint32_t first = __builtin_amdgcn_readfirstlane(start);  // lane 0 is live here
      uint32_t last = end;
      for (int d = 32; d > 0; d >>= 1) last = max(last, (uint32_t)__shfl_xor((int)last, d));
      const uint32_t total = __builtin_amdgcn_readfirstlane(last) - first;
      for (uint32_t t = lane; t < total; t += 64) {
        run_src[wv][t] = e_src[first + t];
        run_wt[wv][t] = e_wt[first + t];
      }
      __builtin_amdgcn_wave_barrier();
      const uint32_t off = live ? start - first : 0u;
      network_sort<T, 16>(run_src[wv], run_wt[wv], off, off + (end - start));
      __builtin_amdgcn_wave_barrier();
      for (uint32_t t = lane; t < total; t += 64) {
        e_src[first + t] = run_src[wv][t];
        e_wt[first + t] = run_wt[wv][t];
      }
    } else {
      network_sort<T, 32>(e_src, e_wt, start, end);
    }
    return;
  }
  // Lists of 33 to 64 entries somewhere in the wave (5 x 5 pooling maps: about fifty): the
  // wave sorts its lists one after the other, a lane per entry, by rank - the number of
  // entries that come before it (by source, then weight, then position) - which is where the
  // entry goes.  Same order as the insertion sort below, which took 5.4 ms for the 524 288
  // lists of a 5 x 5 map on 512 x 1024.
  {
    const uint32_t len = live ? end - start : 0u;
    const uint32_t longest = (uint32_t)wave_max((int)min(len, 0x7fffffffu));
    if (longest > (uint32_t)kNetN && longest <= 64u) {
      const uint32_t lane = threadIdx.x & 63;
      for (int q = 0; q < 64; q++) {
        const uint32_t s = (uint32_t)__builtin_amdgcn_readlane((int)start, q);
        const uint32_t n = (uint32_t)__builtin_amdgcn_readlane((int)len, q);
        if (n < 2u) continue;  // wave-uniform
        const bool mine = lane < n;
        const uint32_t code = e_src[s + (mine ? lane : 0u)];
        const T w = e_wt[s + (mine ? lane : 0u)];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < n; j++) {  // (entry j sits in lane j)
          const uint32_t cj = (uint32_t)__builtin_amdgcn_readlane((int)code, (int)j);
          T wj;
          if constexpr (sizeof(T) == 4) {
            wj = __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w), (int)j));
          } else {
            const long long wb = __builtin_bit_cast(long long, w);
            const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)wb, (int)j);
            const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(wb >> 32), (int)j);
            wj = __builtin_bit_cast(T, (long long)(((unsigned long long)hi << 32) | lo));
          }
          const bool tie = !(wj < w) && !(w < wj);
          rank += (cj < code || (cj == code && (wj < w || (tie && j < lane)))) ? 1u : 0u;
        }
        // (every lane has read the whole list before the first one writes: the stores depend
        // on all of the wave's loads)
        if (mine) {
          e_src[s + rank] = code;
          e_wt[s + rank] = w;
        }
      }
      return;
    }
  }
  if (!live) return;
  if (end - start > kSortMax) return;
  for (uint32_t i = start + 1; i < end; i++) {
    const uint32_t code = e_src[i];
    const T w = e_wt[i];
    uint32_t j = i;
    while (j > start) {
      const uint32_t pc = e_src[j - 1];
      const T pw = e_wt[j - 1];
      // ties (one source reaching the pixel through two corners or points) by weight bits
      if (pc < code || (pc == code && !(pw > w))) break;
      e_src[j] = pc;
      e_wt[j] = pw;
      j--;
    }
    e_src[j] = code;
    e_wt[j] = w;
  }
}

// Planes per thread of the transposed gather's register paths.  The unpoolings read their list
// of about 15 entries once per thread: more planes per thread spread that over more work (8 ->
// 64 planes took a third off the kernel); resampling lists are short: 16 planes measured best
// (0.70 ms against 0.75 with 8 and 0.74 with 32).
template <int OP>
constexpr int planes_per_thread() { return OP == UN_RESAMPLE ? 16 : 64; }

// Smallest value of the wave (all 64 lanes active); see wave_max.
__device__ inline uint32_t wave_min_u32(uint32_t v) {
  constexpr int kId = -1;  // 0xffffffff
  int x = (int)v;
  auto mn = [](int a, int b) { return (int)min((uint32_t)a, (uint32_t)b); };
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x111, 0xf, 0xf, false));  // row_shr:1
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x112, 0xf, 0xf, false));  // row_shr:2
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x114, 0xf, 0xe, false));  // row_shr:4
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x118, 0xf, 0xc, false));  // row_shr:8
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x142, 0xa, 0xf, false));  // row_bcast:15
  x = mn(x, __builtin_amdgcn_update_dpp(kId, x, 0x143, 0xc, 0xf, false));  // row_bcast:31
  return (uint32_t)__builtin_amdgcn_readlane(x, 63);
}

// The unpoolings through LDS windows (fp32; see window_pool for why).  A wave's 64 destination
// pixels read, through their lists, a few short runs of source elements - one per source row
// under a pooling map.  The runs are found greedily on the list entries themselves, as
// intervals of the linear source index (so neither the width of the source nor a seam
// matters): the smallest entry not yet covered starts an interval of kUnIvLen elements, up to
// kUnIntervals of them.  Per plane the intervals are copied to LDS with 16-byte loads and the
// list entries read LDS; for max unpooling the recorded winners travel the same way, their low
// words only (the caller guarantees that every tap code fits 32 bits, and the indices are
// those mapped_max_pool wrote: a tap code or -1).  The sum keeps the order of the list.
// Returns false (wave-uniform) when the wave's lists do not fit; nothing is written then.
constexpr int kUnList = 16;      // entries per lane
constexpr int kUnIntervals = 4;
constexpr int kUnIvLen = 128;    // elements
constexpr int kUnChunks = kUnIntervals * kUnIvLen / 4;  // 16-byte chunks of a window

template <typename T, int OP>
__device__ inline bool window_unpool(const T *__restrict__ src, const int64_t *__restrict__ idx,
                                     T *__restrict__ dst, const uint32_t *__restrict__ e_src,
                                     const T *__restrict__ e_wt, uint32_t start, uint32_t len,
                                     bool live, int p, int64_t plane0, int nc, int nsrc, int ndst,
                                     int K, int idx_scale) {
  if constexpr (sizeof(T) != 4) {
    return false;
  } else {
    constexpr int kDepth = OP == UN_MAX ? 2 : 4;  // planes whose loads are in flight
    constexpr unsigned kZeroOff = kUnChunks * 16;
    __shared__ uint4 win[kThreads / 64][2][kUnChunks + 1];
    __shared__ uint4 iwin[OP == UN_MAX ? kThreads / 64 : 1][2][OP == UN_MAX ? kUnChunks + 1 : 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (__builtin_amdgcn_ballot_w64(len > (uint32_t)kUnList) != 0) return false;
    uint32_t longest = (uint32_t)wave_max((int)len);
    if (longest == 0) return false;

    uint32_t loc[kUnList], want[kUnList];
    T w[kUnList];
#pragma unroll
    for (int u = 0; u < kUnList; u++) {
      const bool in = (uint32_t)u < len;
      const uint32_t cd = e_src[in ? start + u : (len ? start : 0u)];
      w[u] = in ? e_wt[start + u] : T(0);
      loc[u] = in ? (OP == UN_MAX ? cd / (uint32_t)K : cd) : 0xffffffffu;
      want[u] = in ? cd * (uint32_t)idx_scale : 0xffffffffu;  // (no recorded winner reads so)
    }
    // intervals: the smallest entry not yet covered starts the next one
    uint32_t iv[kUnIntervals];
    uint32_t bound = 0;
    int nint = 0;
#pragma unroll
    for (int s2 = 0; s2 < kUnIntervals; s2++) {
      uint32_t m = 0xffffffffu;
#pragma unroll
      for (int u = 0; u < kUnList; u++) m = min(m, loc[u] >= bound ? loc[u] : 0xffffffffu);
      const uint32_t first = wave_min_u32(m);
      iv[s2] = 0xffffffffu;
      if (first != 0xffffffffu) {  // wave-uniform
        iv[s2] = first & ~3u;
        bound = iv[s2] + kUnIvLen;
        nint = s2 + 1;
      } else {
        bound = 0xffffffffu;
      }
    }
    {  // anything left beyond the last interval?
      bool more = false;
#pragma unroll
      for (int u = 0; u < kUnList; u++) more = more || (loc[u] != 0xffffffffu && loc[u] >= bound);
      if (bound != 0xffffffffu && __builtin_amdgcn_ballot_w64(more) != 0) return false;
    }
    // LDS byte offset of every entry (the zero chunk for the padding of a shorter list)
    unsigned off[kUnList];
#pragma unroll
    for (int u = 0; u < kUnList; u++) {
      unsigned sel = 0;
      uint32_t base = iv[0];
#pragma unroll
      for (int s2 = 1; s2 < kUnIntervals; s2++) {
        const bool ge = loc[u] >= iv[s2];  // (unused intervals start at 0xffffffff)
        sel = ge ? (unsigned)s2 : sel;
        base = ge ? iv[s2] : base;
      }
      off[u] = loc[u] == 0xffffffffu ? kZeroOff : (sel * kUnIvLen + (loc[u] - base)) * 4u;
    }
    // the chunks this lane copies per plane: first element, or none
    unsigned goff[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int q = lane + j * 64, s2 = q >> 5;
      uint32_t first = iv[0];
#pragma unroll
      for (int t = 1; t < kUnIntervals; t++) first = s2 == t ? iv[t] : first;
      const uint32_t elem = first + (uint32_t)(q & 31) * 4u;
      goff[j] = (s2 < nint && elem < (uint32_t)nsrc) ? elem * 4u : kOobOffset;
    }
    if (lane < 2) {
      win[wave][lane][kUnChunks] = make_uint4(0u, 0u, 0u, 0u);
      if (OP == UN_MAX) iwin[wave][lane][kUnChunks] = make_uint4(0u, 0u, 0u, 0u);
    }

    const unsigned src_bytes = (unsigned)nsrc * 4u;
    uint4 pre[kDepth][2];
    uint4 ipre[OP == UN_MAX ? kDepth : 1][OP == UN_MAX ? 2 : 1][2];
    auto fetch = [&](int c, int slot) {
      const plane_buf_t pl = plane_buf(src + (plane0 + c) * nsrc, src_bytes);
#pragma unroll
      for (int j = 0; j < 2; j++)
        pre[slot][j] = __builtin_bit_cast(
            uint4, __builtin_amdgcn_raw_buffer_load_b128(pl, (int)goff[j], 0, 0));
      if constexpr (OP == UN_MAX) {
        // (an index plane of 8-byte elements: the same chunk is two 16-byte loads; offsets
        // beyond 4 GiB are ruled out by the caller)
        const plane_buf_t ipl = plane_buf(idx + (plane0 + c) * nsrc, (unsigned)nsrc * 8u);
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const unsigned o = goff[j] == kOobOffset ? kOobOffset : goff[j] * 2u;
          ipre[slot][j][0] = __builtin_bit_cast(
              uint4, __builtin_amdgcn_raw_buffer_load_b128(ipl, (int)o, 0, 0));
          ipre[slot][j][1] = __builtin_bit_cast(
              uint4, __builtin_amdgcn_raw_buffer_load_b128(ipl, (int)(o == kOobOffset ? o : o + 16u),
                                                           0, 0));
        }
      }
    };
    auto stash = [&](int slot, int buf) {
      win[wave][buf][lane] = pre[slot][0];
      win[wave][buf][lane + 64] = pre[slot][1];
      if constexpr (OP == UN_MAX) {
#pragma unroll
        for (int j = 0; j < 2; j++)
          iwin[wave][buf][lane + 64 * j] = make_uint4(ipre[slot][j][0].x, ipre[slot][j][0].z,
                                                      ipre[slot][j][1].x, ipre[slot][j][1].z);
      }
      __builtin_amdgcn_wave_barrier();
    };
    auto compute = [&](int c, int buf) {
      const char *wb = reinterpret_cast<const char *>(&win[wave][buf][0]);
      const char *ib = reinterpret_cast<const char *>(&iwin[OP == UN_MAX ? wave : 0][buf][0]);
      T v[kUnList];
      uint32_t won[kUnList];
#pragma unroll
      for (int u = 0; u < kUnList; u++) {
        v[u] = *reinterpret_cast<const T *>(wb + off[u]);
        if (OP == UN_MAX) won[u] = *reinterpret_cast<const uint32_t *>(ib + off[u]);
      }
      __builtin_amdgcn_sched_barrier(0);
      T a = T(0);
#pragma unroll
      for (int u = 0; u < kUnList; u++) {
        // (padding: weight zero times the zero chunk; max unpooling: its `want` matches nothing)
        if (OP == UN_MAX)
          a = won[u] == want[u] ? mcx_fma(w[u], v[u], a) : a;
        else
          a = mcx_fma(w[u], v[u], a);
      }
      const int cc = min(c, nc - 1);
      buf_store(plane_buf(dst + (plane0 + cc) * ndst, (unsigned)ndst * 4u),
                (live && c < nc) ? (unsigned)p * 4u : kOobOffset, OP == UN_AVG ? a / (T)K : a);
      __builtin_amdgcn_wave_barrier();
    };
#pragma unroll
    for (int u = 0; u < kDepth; u++) fetch(min(u, nc - 1), u);
    stash(0, 0);
    for (int cb = 0; cb < nc; cb += kDepth) {
#pragma unroll
      for (int u = 0; u < kDepth; u++) {
        const int c = cb + u;
        fetch(min(c + kDepth, nc - 1), u);
        compute(c, u & 1);
        stash((u + 1) % kDepth, (u + 1) & 1);
      }
    }
    return true;
  }
}

// Planes [plane0, plane0 + nc) of destination pixel p through its list [start, end).  UN_MAX
// keeps a contribution only where the recorded winner of that source element is this tap.
template <typename T, int OP>
__device__ inline void transposed_gather_planes(
    const T *__restrict__ src, const int64_t *__restrict__ idx, T *__restrict__ dst,
    const uint32_t *__restrict__ e_src, const T *__restrict__ e_wt, uint32_t start, uint32_t end,
    int p, int64_t plane0, int nc, int nsrc, int ndst, int K, int idx_scale, uint32_t longest) {
  constexpr int kTCH = planes_per_thread<OP>();
  const T *s0 = src + plane0 * nsrc;
  const int64_t *i0 = OP == UN_MAX ? idx + plane0 * nsrc : nullptr;
  // Short lists (every lane of the wave has at most kListRegs entries: pooling maps): the
  // list is read once into registers and the planes are walked in the outer loop, so that a
  // plane's few source rows are read in one go and hit in cache; with the planes inside,
  // every sampled byte came from memory.  The additions keep the order of the list.
  constexpr int kListRegs = 24, kGroup = 6;
  const uint32_t len = end - start;
  if (OP != UN_RESAMPLE) {
    // (`longest`: the longest list of the wave, taken by the caller while all 64 lanes were
    // still there)
    T *d0 = dst + plane0 * ndst + p;
    // Lists longer than kListRegs (5 x 5 pooling maps: about fifty entries) take several
    // passes of kListRegs entries over the planes; a pass continues from the sum the pass
    // before left in the destination, so the order of the additions stays that of the list.
    uint32_t base = 0;
    do {
      const uint32_t part = len > base ? len - base : 0u;  // this lane's entries in the pass
      const uint32_t wave_part = longest - base;
      const bool first = base == 0, last = base + kListRegs >= longest;
      // per entry: the source element to load and, for max unpooling, the value the recorded
      // winner must have.  An entry past the end of the lane's list loads the lane's first
      // source element (a valid address) and is dropped by a test, never by its zero weight
      // (an Inf or NaN in an unrelated source element must not reach the destination): the
      // average tests its position, max unpooling is given a winner no element can record.
      uint32_t code[kListRegs], want[OP == UN_MAX ? kListRegs : 1];
      T w[kListRegs];
#pragma unroll
      for (int u = 0; u < kListRegs; u++) {
        const bool in = (uint32_t)u < part;
        const uint32_t cd = e_src[in ? start + base + u : (len ? start : 0u)];
        code[u] = OP == UN_MAX ? cd / (uint32_t)K : cd;
        if constexpr (OP == UN_MAX) want[u] = in ? cd : 0xffffffffu;
        w[u] = in ? e_wt[start + base + u] : T(0);
      }
      for (int c = 0; c < nc; c++) {
        const T *sc = s0 + (int64_t)c * nsrc;
        const int64_t *ic = OP == UN_MAX ? i0 + (int64_t)c * nsrc : nullptr;
        T a = first ? T(0) : d0[(int64_t)c * ndst];
#pragma unroll
        for (int g = 0; g < kListRegs / kGroup; g++) {
          if ((uint32_t)(g * kGroup) < wave_part) {  // wave-uniform, once per six entries
            T v[kGroup];
            bool keep[kGroup];
#pragma unroll
            for (int j = 0; j < kGroup; j++) {
              const uint32_t n = code[g * kGroup + j];
              v[j] = sc[n];
              // (recorded winners are offsets into the map, below 2^31: 0xffffffff * idx_scale
              // equals none of them, nor the -1 of "no winner")
              if constexpr (OP == UN_MAX)
                keep[j] = ic[n] == (int64_t)want[g * kGroup + j] * idx_scale;
              else
                keep[j] = (uint32_t)(g * kGroup + j) < part;
            }
#pragma unroll
            for (int j = 0; j < kGroup; j++)
              if (keep[j]) a = mcx_fma(w[g * kGroup + j], v[j], a);
          }
        }
        d0[(int64_t)c * ndst] = (OP == UN_AVG && last) ? a / (T)K : a;
      }
      base += kListRegs;
    } while (base < longest);
    return;
  }
  if constexpr (OP == UN_RESAMPLE) {
    // Resampling lists are short (three entries on average under a cube map, up to fourteen)
    // and differ in length from lane to lane.  Every lane walks the wave's longest list
    // without a branch: an entry past the end of a lane's list loads out of range (a zero, no
    // memory traffic) with weight zero, so that all loads of a step are in flight together.
    // (With the loads behind the per-lane test every load was followed by a full wait: 0.93 ms
    // at 4 x 64 planes of 512 x 1024, against 0.70 ms.  What remains is the texture path, busy
    // 80 % of the time: the padded entries cost it as much as real ones, and the longest list
    // of a wave is 4.9 entries where the average is 3.0.)
    if ((int64_t)nsrc * (int64_t)sizeof(T) < (int64_t)kOobOffset) {
      constexpr int kPair = 2;
      plane_buf_t pl[kTCH];
#pragma unroll
      for (int c = 0; c < kTCH; c++)
        pl[c] = plane_buf(s0 + (int64_t)min(c, nc - 1) * nsrc, (unsigned)nsrc * (unsigned)sizeof(T));
      T acc[kTCH];
#pragma unroll
      for (int c = 0; c < kTCH; c++) acc[c] = T(0);
      const uint32_t len = end - start;
      constexpr int kRegs = 8, kStep = 4;
      if (longest <= (uint32_t)kRegs) {
        // the whole list first (one round trip), then the samples, four entries at a time
        unsigned off[kRegs];
        T w[kRegs];
#pragma unroll
        for (int u = 0; u < kRegs; u++) {
          const bool in = (uint32_t)u < len;
          const uint32_t ee = in ? start + u : 0u;
          const uint32_t code = e_src[ee];
          const T wt = e_wt[ee];
          off[u] = in ? code * (unsigned)sizeof(T) : kOobOffset;
          w[u] = in ? wt : T(0);
        }
#pragma unroll
        for (int g = 0; g < kRegs / kStep; g++) {
          if ((uint32_t)(g * kStep) < longest) {  // wave-uniform
            T v[kStep][kTCH];
#pragma unroll
            for (int u = 0; u < kStep; u++)
#pragma unroll
              for (int c = 0; c < kTCH; c++) v[u][c] = buf_load(pl[c], off[g * kStep + u], T());
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kStep; u++)
#pragma unroll
              for (int c = 0; c < kTCH; c++)
                acc[c] = mcx_fma(w[g * kStep + u], v[u][c], acc[c]);
          }
        }
      } else {
        for (uint32_t t = 0; t < longest; t += kPair) {
          unsigned off[kPair];
          T w[kPair];
#pragma unroll
          for (int u = 0; u < kPair; u++) {
            const bool in = t + u < len;
            const uint32_t ee = in ? start + t + u : 0u;
            const uint32_t code = e_src[ee];
            const T wt = e_wt[ee];
            off[u] = in ? code * (unsigned)sizeof(T) : kOobOffset;
            w[u] = in ? wt : T(0);
          }
          T v[kPair][kTCH];
#pragma unroll
          for (int u = 0; u < kPair; u++)
#pragma unroll
            for (int c = 0; c < kTCH; c++) v[u][c] = buf_load(pl[c], off[u], T());
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < kPair; u++)
#pragma unroll
            for (int c = 0; c < kTCH; c++) acc[c] = mcx_fma(w[u], v[u][c], acc[c]);
        }
      }
      T *d0 = dst + plane0 * ndst + p;
#pragma unroll
      for (int c = 0; c < kTCH; c++)
        if (c < nc) d0[(int64_t)c * ndst] = acc[c];
      return;
    }
  }
  T acc[kTCH];
#pragma unroll
  for (int c = 0; c < kTCH; c++) acc[c] = T(0);
  // kUnroll entries per trip so that their loads are in flight together; entries past
  // the end repeat the last valid one and are dropped (by a test, not by a zero weight: an Inf
  // or NaN in an unrelated source element must not reach the destination).
  constexpr int kUnroll = OP == UN_RESAMPLE ? 2 : 4;
  for (uint32_t e = start; e < end; e += kUnroll) {
    uint32_t code[kUnroll];
    T w[kUnroll];
    bool in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      in[u] = e + u < end;
      const uint32_t ee = in[u] ? e + u : e;
      code[u] = e_src[ee];
      w[u] = e_wt[ee];
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const uint32_t n = OP == UN_MAX ? code[u] / (uint32_t)K : code[u];
      const int64_t want = (int64_t)code[u] * idx_scale;
#pragma unroll
      for (int c = 0; c < kTCH; c++) {
        if (c >= nc) continue;
        if (OP == UN_MAX) {
          const bool hit = i0[(int64_t)c * nsrc + n] == want;
          if (in[u] & hit) acc[c] = mcx_fma(w[u], s0[(int64_t)c * nsrc + n], acc[c]);
        } else {
          if (in[u]) acc[c] = mcx_fma(w[u], s0[(int64_t)c * nsrc + n], acc[c]);
        }
      }
    }
  }
  T *d0 = dst + plane0 * ndst + p;
#pragma unroll
  for (int c = 0; c < kTCH; c++)
    if (c < nc) d0[(int64_t)c * ndst] = OP == UN_AVG ? acc[c] / (T)K : acc[c];
}

// One workgroup: 256 destination pixels x `reps` groups of kTCH planes.
template <typename T, int OP>
__global__ __launch_bounds__(kThreads, OP == UN_AVG ? 4 : OP == UN_MAX ? 3 : 1) void transposed_gather_kernel(
    const T *__restrict__ src, const int64_t *__restrict__ idx, T *__restrict__ dst,
    const uint32_t *__restrict__ local, const uint32_t *__restrict__ bsum,
    const uint32_t *__restrict__ e_src, const T *__restrict__ e_wt, int64_t planes, int nsrc,
    int ndst, int K, int idx_scale, int groups, int reps, int windows) {
  constexpr int kTCH = planes_per_thread<OP>();
  // (the unpoolings: every XCD takes one contiguous run of the destination, so that the source
  // rows neighbouring destination rows share are read into one L2 only)
  const int wg = OP == UN_RESAMPLE ? (int)blockIdx.x : xcd_contiguous(blockIdx.x, gridDim.x);
  const int pg = wg % groups;
  const int p = (wg / groups) * kThreads + threadIdx.x;
  const bool live = p < ndst;
  const int pc = live ? p : 0;
  const uint32_t start = local[pc] + bsum[pc / kScanBlock];
  const uint32_t end = local[pc + 1] + bsum[(pc + 1) / kScanBlock];
  const int64_t first_plane = (int64_t)pg * reps * kTCH;
  const int np = (int)min((int64_t)reps * kTCH, planes - first_plane);
  if constexpr (OP != UN_RESAMPLE) {
    if (windows && window_unpool<T, OP>(src, idx, dst, e_src, e_wt, start, live ? end - start : 0u,
                                        live, p, first_plane, np, nsrc, ndst, K, idx_scale))
      return;
  }
  const uint32_t longest = (uint32_t)wave_max(live ? (int)(end - start) : 0);
  if (!live) return;
  for (int done = 0; done < np; done += kTCH)
    transposed_gather_planes<T, OP>(src, idx, dst, e_src, e_wt, start, end, p,
                                    first_plane + done, min(kTCH, np - done), nsrc, ndst, K,
                                    idx_scale, longest);
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
                  int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t MH, int64_t MW, int64_t K,
                  int64_t P, int interp, hipStream_t s) {
  const int64_t N = MH * MW;
  // (the same test as in direct_gather: unweighted pooling with at most 9 taps)
  const bool tap_registers = OP != OP_RESAMPLE && P == 0;
  int cpt = tap_registers ? kPoolCH : kCH;
  if (tap_registers && B * C <= 0x7fffffffLL) {
    // Images and channels are one run of planes to these kernels, and resolving a thread's
    // taps costs as much as sampling some fifty planes: every thread takes as many planes
    // as still leaves about eight waves for each of the 1024 SIMDs.
    C *= B;
    B = 1;
    const int64_t waves = (int64_t)div_up(MW, Patch<OP>::kW) * div_up(MH, Patch<OP>::kH) *
                          (kThreads / 64);
    while (cpt < 1024 && cpt * 2 <= C && waves * div_up(C, cpt * 2) >= 8192) cpt *= 2;
  }
  // Unweighted resampling: every thread walks a run of planes with a ring of loads in flight.
  // (images and channels are one run of planes, kCH of them per thread: longer runs measured
  // slower, 0.321 / 0.330 / 0.332 / 0.350 ms at 8 / 16 / 32 / 64 planes for 256 planes of
  // 512 x 1024 sampled at 256 x 1536 locations)
  // (the planes go into the grid's second dimension, which holds 65535 workgroups: beyond
  // that the images stay in the third)
  const bool plane_ring = OP == OP_RESAMPLE && P == 0 && K == 1 && B * C <= 0x7fffffffLL &&
                          N * 8 < (int64_t)kOobOffset && (B * C + cpt - 1) / cpt <= 65535;
  if (plane_ring) {
    C *= B;
    B = 1;
  }
  if ((C + cpt - 1) / cpt > 65535) return MCX_E_SHAPE;
  dim3 grid(div_up(MW, Patch<OP>::kW) * div_up(MH, Patch<OP>::kH), div_up(C, cpt), (unsigned)B);
  // (the LDS-window path copies 16-byte chunks of source rows)
  const int windows = plane_ring || (tap_registers && K <= 9 && N * 8 < (int64_t)kOobOffset &&
                                     IW % (16 / (int)sizeof(T)) == 0 &&
                                     (reinterpret_cast<uintptr_t>(in) & 15) == 0)
                          ? 1
                          : 0;
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((gather_kernel<T, MODE, OP>), grid, dim3(kThreads),
                                               0, s, (const T *)in, (const T *)map,
                                               (const T *)iw, (T *)out, idx, (int)C, (int)IH,
                                               (int)IW, (int)N, (int)MW, (int)K, (int)P, cpt,
                                               windows));
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}


// Workspace of the transposed-map form.  `samples` = source locations x taps x
// points; every sample can land on `corners` destination pixels.
struct TransposedLayout {
  size_t local, cursor, bsum, e_src, e_wt, total;
  int nblocks;
  bool ok;
};

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

TransposedLayout transposed_layout(int64_t ndst, int64_t samples, int corners, size_t elem) {
  TransposedLayout l{};
  const int64_t cap = samples * corners;
  l.ok = ndst > 0 && samples > 0 && cap <= 0x7fffffffLL && ndst < 0x7fffffffLL;
  if (!l.ok) return l;
  l.nblocks = (int)((ndst + 1 + kScanBlock - 1) / kScanBlock);
  size_t off = 0;
  l.local = off;  off += align256((size_t)(ndst + 1) * 4);
  l.cursor = off; off += align256((size_t)ndst * 4);
  l.bsum = off;   off += align256((size_t)l.nblocks * 4);
  l.e_src = off;  off += align256((size_t)cap * 4);
  l.e_wt = off;   off += align256((size_t)cap * elem);
  l.total = off;
  return l;
}

inline int corners_of(int interp) { return canonical_interp(interp) == kInterpNearest ? 1 : 4; }

// Returns -1000 when the form does not apply (no or short workspace, sizes beyond
// 32-bit entry indices): the caller then runs the atomic scatter instead.
constexpr int kNotApplicable = -1000;

// Builds the compressed transposed map of `map` into `ws` (count -> prefix sum -> fill ->
// per-pixel sort).  `max_codes`: an entry's source code is (location * K + tap), which max
// unpooling needs to test the recorded winner; otherwise it is the location alone.
// Returns kNotApplicable when the form does not apply.
template <typename T>
int build_transposed(const void *map, const void *iw, void *ws, size_t ws_bytes, int64_t nsrc,
                     int64_t K, int64_t P, int64_t DH, int64_t DW, int interp, bool max_codes,
                     hipStream_t s) {
  const int64_t pm = P ? P : 1;
  const int64_t samples = nsrc * K * pm, ndst = DH * DW;
  const TransposedLayout l = transposed_layout(ndst, samples, corners_of(interp), sizeof(T));
  if (!ws || !l.ok || ws_bytes < l.total || nsrc * K > 0xffffffffLL) return kNotApplicable;
  char *base = (char *)ws;
  uint32_t *local = (uint32_t *)(base + l.local), *cursor = (uint32_t *)(base + l.cursor);
  uint32_t *bsum = (uint32_t *)(base + l.bsum), *e_src = (uint32_t *)(base + l.e_src);
  T *e_wt = (T *)(base + l.e_wt);
  int rc = fill<uint32_t>(local, ndst + 1, 0u, s);
  if (rc) return rc;
  if ((rc = fill<uint32_t>(cursor, ndst, 0u, s))) return rc;
  const int per_code = (int)(max_codes ? pm : pm * K);
  const dim3 sgrid(div_up(nsrc, kThreads)), blk(kThreads);
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((transposed_map_kernel<T, MODE, false>), sgrid, blk,
                                               0, s, (const T *)map, (const T *)iw, nsrc,
                                               (int)(K * pm), per_code, (int)DH, (int)DW, local,
                                               cursor, bsum, e_src, e_wt));
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(scan_blocks_kernel, dim3(l.nblocks), blk, 0, s, local, bsum, ndst + 1);
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL(scan_sums_kernel, dim3(1), blk, 0, s, bsum, l.nblocks);
  MCX_HIP_CHECK_LAUNCH();
  // (the fill's atomics return a value: 64 of them on neighbouring counters are served one
  // after the other - 0.14 against 0.09 ms - so it keeps one thread per sample)
  const dim3 fgrid(div_up(samples, kThreads));
  MCX_DISPATCH_MODE(interp, hipLaunchKernelGGL((transposed_map_kernel<T, MODE, true>), fgrid, blk,
                                               0, s, (const T *)map, (const T *)iw, samples, 1,
                                               per_code, (int)DH, (int)DW, local, cursor, bsum,
                                               e_src, e_wt));
  MCX_HIP_CHECK_LAUNCH();
  hipLaunchKernelGGL((sort_entries_kernel<T>), dim3(div_up(ndst, kThreads)), blk, 0, s, local, bsum,
                     e_src, e_wt, (int)ndst);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

// The gather through a built transposed map (in `ws`: a call's workspace or a caller's plan).
template <typename T, int OP>
int gather_transposed(const void *src, const int64_t *idx, void *dst, const void *ws,
                      size_t ws_bytes, int64_t planes, int64_t nsrc, int64_t K, int64_t P,
                      int64_t DH, int64_t DW, int interp, hipStream_t s) {
  const int64_t pm = P ? P : 1;
  const int64_t samples = nsrc * K * pm, ndst = DH * DW;
  const TransposedLayout l = transposed_layout(ndst, samples, corners_of(interp), sizeof(T));
  if (!ws || !l.ok || ws_bytes < l.total || nsrc * K > 0xffffffffLL) return kNotApplicable;
  constexpr int kTCH = planes_per_thread<OP>();
  // The LDS-window path copies 16-byte chunks of source planes (fp32; for max unpooling the
  // recorded winners too, compared by their low words: every tap code must fit 32 bits).
  const bool windows = OP != UN_RESAMPLE && sizeof(T) == 4 && nsrc % 4 == 0 &&
                       (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
                       nsrc * 8 < (int64_t)kOobOffset && ndst * 4 < (int64_t)kOobOffset &&
                       (OP != UN_MAX || ((reinterpret_cast<uintptr_t>(idx) & 15) == 0 &&
                                         nsrc * K * pm * 2 < 0xffffffffLL));
  // A workgroup takes `reps` groups of kTCH planes (a wave's window set-up is spread over
  // them) while about eight waves per SIMD remain.
  int reps = 1;
  const int64_t tiles = (ndst + kThreads - 1) / kThreads;
  while (windows && reps < 4 && (int64_t)reps * 2 * kTCH <= planes &&
         tiles * (kThreads / 64) * ((planes + reps * 2 * kTCH - 1) / (reps * 2 * kTCH)) >= 8192)
    reps *= 2;
  const int64_t groups = (planes + reps * kTCH - 1) / (reps * kTCH);
  const int64_t blocks = groups * tiles;
  if (blocks > 0x7fffffffLL) return kNotApplicable;
  const char *base = (const char *)ws;
  hipLaunchKernelGGL((transposed_gather_kernel<T, OP>), dim3((unsigned)blocks), dim3(kThreads), 0,
                     s, (const T *)src, idx, (T *)dst, (const uint32_t *)(base + l.local),
                     (const uint32_t *)(base + l.bsum), (const uint32_t *)(base + l.e_src),
                     (const T *)(base + l.e_wt), planes, (int)nsrc, (int)ndst, (int)K,
                     (int)(pm * 2), (int)groups, reps, windows ? 1 : 0);
  MCX_HIP_CHECK_LAUNCH();
  return 0;
}

template <typename T, int OP>
int launch_transposed(const void *src, const int64_t *idx, const void *map, const void *iw,
                      void *dst, void *ws, size_t ws_bytes, int64_t planes, int64_t nsrc,
                      int64_t K, int64_t P, int64_t DH, int64_t DW, int interp, hipStream_t s) {
  const int64_t groups = (planes + planes_per_thread<OP>() - 1) / planes_per_thread<OP>();
  if (groups * ((DH * DW + kThreads - 1) / kThreads) > 0x7fffffffLL) return kNotApplicable;
  const int rc = build_transposed<T>(map, iw, ws, ws_bytes, nsrc, K, P, DH, DW, interp,
                                     OP == UN_MAX, s);
  if (rc) return rc;
  return gather_transposed<T, OP>(src, idx, dst, ws, ws_bytes, planes, nsrc, K, P, DH, DW, interp,
                                  s);
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

// Samples are addressed with 32-bit byte offsets inside a plane (see plane_buf).
bool plane_beyond_4gib(int64_t pixels, int dtype) {
  return pixels * (dtype == MCX_F64 ? 8 : 4) > (int64_t)kOobOffset;
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
  if (bad_dims({B, C, SH, SW, MH, MW, SH * SW, MH * MW, MH * MW * (P ? P : 1) * 2}) || B > 65535 ||
      plane_beyond_4gib(SH * SW, dtype))
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_RESAMPLE>(src, map, iw, dst, nullptr, B, C, SH, SW, MH, MW, 1,
                                             P, interp, s);
  return launch_gather<double, OP_RESAMPLE>(src, map, iw, dst, nullptr, B, C, SH, SW, MH, MW, 1,
                                            P, interp, s);
}

namespace {
template <typename T>
int resample_to_map_t(const void *in, const void *map, const void *iw, void *out, void *ws,
                      size_t ws_bytes, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                      int64_t OW, int64_t P, int interp, hipStream_t s) {
  const int rc = launch_transposed<T, UN_RESAMPLE>(in, nullptr, map, iw, out, ws, ws_bytes, B * C,
                                                   IH * IW, 1, P, OH, OW, interp, s);
  if (rc != kNotApplicable) return rc;
  return launch_scatter<T, OP_RESAMPLE>(in, map, iw, out, B, C, OH, OW, IH * IW, 1, P, interp, s);
}

size_t transposed_workspace(int64_t nsrc, int64_t K, int64_t P, int64_t DH, int64_t DW, int interp,
                            int dtype) {
  if (dtype != MCX_F32 && dtype != MCX_F64) return 0;
  if (bad_dims({nsrc, K, DH, DW, DH * DW}) || P < 0) return 0;
  const TransposedLayout l = transposed_layout(DH * DW, nsrc * K * (P ? P : 1), corners_of(interp),
                                               dtype == MCX_F32 ? 4 : 8);
  return l.ok ? l.total : 0;
}
}  // namespace

extern "C" size_t mcx_resample_to_map_workspace(int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                                                int64_t P, int interp, int dtype) {
  if (bad_dims({IH, IW, IH * IW})) return 0;
  return transposed_workspace(IH * IW, 1, P, OH, OW, interp, dtype);
}

extern "C" size_t mcx_unpool_workspace(int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                       int64_t P, int interp, int dtype) {
  if (bad_dims({OH, OW, OH * OW})) return 0;
  return transposed_workspace(OH * OW, K, P, IH, IW, interp, dtype);
}

extern "C" int mcx_resample_to_map(const void *in, const void *map, const void *iw, void *out,
                                   void *workspace, size_t workspace_bytes, int64_t B, int64_t C,
                                   int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t P,
                                   int interp, int dtype, void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, IH * IW, OH * OW, IH * IW * (P ? P : 1) * 2}) || B > 65535)
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return resample_to_map_t<float>(in, map, iw, out, workspace, workspace_bytes, B, C, IH, IW, OH,
                                    OW, P, interp, s);
  return resample_to_map_t<double>(in, map, iw, out, workspace, workspace_bytes, B, C, IH, IW, OH,
                                   OW, P, interp, s);
}

extern "C" int mcx_max_pool(const void *in, const void *map, const void *iw, void *out,
                            int64_t *idx, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                            int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                            void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (!idx) return MCX_E_NULL;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535 ||
      plane_beyond_4gib(IH * IW, dtype))
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_MAX>(in, map, iw, out, idx, B, C, IH, IW, OH, OW, K, P, interp,
                                        s);
  return launch_gather<double, OP_MAX>(in, map, iw, out, idx, B, C, IH, IW, OH, OW, K, P, interp,
                                       s);
}

extern "C" int mcx_avg_pool(const void *in, const void *map, const void *iw, void *out, int64_t B,
                            int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                            int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(in, map, iw, out, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535 ||
      plane_beyond_4gib(IH * IW, dtype))
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_gather<float, OP_AVG>(in, map, iw, out, nullptr, B, C, IH, IW, OH, OW, K, P,
                                        interp, s);
  return launch_gather<double, OP_AVG>(in, map, iw, out, nullptr, B, C, IH, IW, OH, OW, K, P,
                                       interp, s);
}

namespace {
template <typename T>
int avg_unpool_t(const void *gout, const void *map, const void *iw, void *gin, void *ws,
                 size_t ws_bytes, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                 int64_t OW, int64_t K, int64_t P, int interp, hipStream_t s) {
  const int rc = launch_transposed<T, UN_AVG>(gout, nullptr, map, iw, gin, ws, ws_bytes, B * C,
                                              OH * OW, K, P, IH, IW, interp, s);
  if (rc != kNotApplicable) return rc;
  return launch_scatter<T, OP_AVG>(gout, map, iw, gin, B, C, IH, IW, OH * OW, K, P, interp, s);
}
}  // namespace

extern "C" int mcx_avg_unpool(const void *gout, const void *map, const void *iw, void *gin,
                              void *workspace, size_t workspace_bytes, int64_t B, int64_t C,
                              int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                              int interp, int dtype, void *stream) {
  if (int rc = check_common(gout, map, iw, gin, P, dtype)) return rc;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) || B > 65535) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return avg_unpool_t<float>(gout, map, iw, gin, workspace, workspace_bytes, B, C, IH, IW, OH, OW,
                               K, P, interp, s);
  return avg_unpool_t<double>(gout, map, iw, gin, workspace, workspace_bytes, B, C, IH, IW, OH, OW,
                              K, P, interp, s);
}

namespace {
template <typename T>
int launch_max_unpool(const void *gout, const int64_t *idx, const void *map, const void *iw,
                      void *gin, void *ws, size_t ws_bytes, int64_t B, int64_t C, int64_t IH,
                      int64_t IW, int64_t N, int64_t K, int64_t P, int interp, hipStream_t s) {
  int rc = launch_transposed<T, UN_MAX>(gout, idx, map, iw, gin, ws, ws_bytes, B * C, N, K, P, IH,
                                        IW, interp, s);
  if (rc != kNotApplicable) return rc;
  rc = mcx::fill<T>((T *)gin, B * C * IH * IW, T(0), s);
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
                              const void *iw, void *gin, void *workspace, size_t workspace_bytes,
                              int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                              int64_t K, int64_t P, int interp, int dtype, void *stream) {
  if (int rc = check_common(gout, map, iw, gin, P, dtype)) return rc;
  if (!idx) return MCX_E_NULL;
  if (bad_dims({B, C, IH, IW, OH, OW, K, IH * IW, OH * OW}) ||
      B * C * OH * OW > (int64_t)0x7fffffff * kThreads)
    return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MCX_F32)
    return launch_max_unpool<float>(gout, idx, map, iw, gin, workspace, workspace_bytes, B, C, IH,
                                    IW, OH * OW, K, P, interp, s);
  return launch_max_unpool<double>(gout, idx, map, iw, gin, workspace, workspace_bytes, B, C, IH,
                                   IW, OH * OW, K, P, interp, s);
}

// ---- scatter plans: the transposed map of one sample map, built once -------------------
extern "C" size_t mcx_scatter_plan_bytes(int64_t MH, int64_t MW, int64_t DH, int64_t DW, int64_t K,
                                         int64_t P, int interp, int dtype) {
  if (bad_dims({MH, MW, MH * MW, K})) return 0;
  return transposed_workspace(MH * MW, K, P, DH, DW, interp, dtype);
}

extern "C" int mcx_scatter_plan_build(const void *map, const void *iw, void *plan,
                                      size_t plan_bytes, mcx_plan_desc *desc, int64_t MH,
                                      int64_t MW, int64_t DH, int64_t DW, int64_t K, int64_t P,
                                      int interp, int dtype, int for_max_unpool, void *stream) {
  if (dtype != MCX_F32 && dtype != MCX_F64) return MCX_E_DTYPE;
  if (!map || !plan || !desc || (P > 0) != (iw != nullptr)) return MCX_E_NULL;
  if (bad_dims({MH, MW, DH, DW, K, MH * MW, DH * DW}) || P < 0) return MCX_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  desc->magic = 0;  // (not a plan until the build has been enqueued)
  const int rc = dtype == MCX_F32
                     ? build_transposed<float>(map, iw, plan, plan_bytes, MH * MW, K, P, DH, DW,
                                               interp, for_max_unpool != 0, s)
                     : build_transposed<double>(map, iw, plan, plan_bytes, MH * MW, K, P, DH, DW,
                                                interp, for_max_unpool != 0, s);
  if (rc) return rc == kNotApplicable ? MCX_E_WORKSPACE : rc;
  mcx::plan_desc_fill(desc, for_max_unpool ? MCX_PLAN_SCATTER_MAX : MCX_PLAN_SCATTER, interp, dtype,
                      DH, DW, MH, MW, K, P, plan,
                      transposed_workspace(MH * MW, K, P, DH, DW, interp, dtype), map, iw);
  return 0;
}

namespace {
template <int OP>
int planned_gather(const void *src, const int64_t *idx, void *dst, const void *plan,
                   size_t plan_bytes, const mcx_plan_desc *desc, int64_t B, int64_t C, int64_t SH,
                   int64_t SW, int64_t DH, int64_t DW, int64_t K, int64_t P, int interp, int dtype,
                   void *stream) {
  if (dtype != MCX_F32 && dtype != MCX_F64) return MCX_E_DTYPE;
  if (!src || !dst || !plan || (OP == UN_MAX && !idx)) return MCX_E_NULL;
  if (bad_dims({B, C, SH, SW, DH, DW, K, SH * SW, DH * DW}) || P < 0 || B > 65535)
    return MCX_E_SHAPE;
  // the plan must be the one built for this op (a max-unpool plan's source codes differ from
  // the others'), interpolation, sizes and data type, at this address
  if (int rc = mcx::plan_desc_check(desc, OP == UN_MAX ? MCX_PLAN_SCATTER_MAX : MCX_PLAN_SCATTER,
                                    interp, dtype, DH, DW, SH, SW, K, P, plan, plan_bytes, false,
                                    nullptr, nullptr))
    return rc;
  hipStream_t s = (hipStream_t)stream;
  const int rc = dtype == MCX_F32
                     ? gather_transposed<float, OP>(src, idx, dst, plan, plan_bytes, B * C, SH * SW,
                                                    K, P, DH, DW, interp, s)
                     : gather_transposed<double, OP>(src, idx, dst, plan, plan_bytes, B * C,
                                                     SH * SW, K, P, DH, DW, interp, s);
  return rc == kNotApplicable ? MCX_E_WORKSPACE : rc;
}
}  // namespace

extern "C" int mcx_resample_to_map_planned(const void *in, const void *plan, size_t plan_bytes,
                                           const mcx_plan_desc *desc, void *out, int64_t B,
                                           int64_t C, int64_t IH, int64_t IW, int64_t OH,
                                           int64_t OW, int64_t P, int interp, int dtype,
                                           void *stream) {
  return planned_gather<UN_RESAMPLE>(in, nullptr, out, plan, plan_bytes, desc, B, C, IH, IW, OH, OW, 1, P,
                                     interp, dtype, stream);
}

extern "C" int mcx_avg_unpool_planned(const void *gout, const void *plan, size_t plan_bytes,
                                      const mcx_plan_desc *desc, void *gin, int64_t B, int64_t C,
                                      int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                      int64_t P, int interp, int dtype, void *stream) {
  return planned_gather<UN_AVG>(gout, nullptr, gin, plan, plan_bytes, desc, B, C, OH, OW, IH, IW, K, P,
                                interp, dtype, stream);
}

extern "C" int mcx_max_unpool_planned(const void *gout, const int64_t *idx, const void *plan,
                                      size_t plan_bytes, const mcx_plan_desc *desc, void *gin,
                                      int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                                      int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                      void *stream) {
  return planned_gather<UN_MAX>(gout, idx, gin, plan, plan_bytes, desc, B, C, OH, OW, IH, IW, K, P, interp,
                                dtype, stream);
}
