// extern "C" entry points of the mapped (transposed) convolution.  Validates the
// arguments, then routes each of the three products (gather-product,
// product-scatter, weight gradient; see mcx_conv_generic.hip for the roles) to the
// matrix-core kernels when they cover the case (fp32 and bf16 storage, at most 4
// interpolation points per tap) and to the scalar kernels otherwise (fp64, or fp32
// with more points).
#include <algorithm>
#include <initializer_list>
#include <mutex>

#include "mcx.h"
#include "mcx_conv.h"
#include "mcx_plan.h"
#include "mcx_taps.h"

using namespace mcx;

// Scratch of mcx_conv_forward_static: one array per GPU, part of the loaded code object, so
// the entry point never allocates.  Host code must not use the array's name as an address
// (it is a host-side stand-in); the device address is looked up once per device with
// hipGetSymbolAddress and kept in g_static_scratch.
constexpr size_t kStaticScratchBytes = MCX_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
void *g_static_scratch[kMaxDevices] = {};
std::mutex g_static_scratch_mutex;

// Device address of `scratch` on the current device (looked up at the first call on that
// device); nullptr and *rc set on failure.
void *static_scratch_of_current_device(int *rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    *rc = (int)e;
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    *rc = MCX_E_SHAPE;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      *rc = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
      return nullptr;
    }
    g_static_scratch[dev] = ptr;
  }
  return g_static_scratch[dev];
}

// A timing request (mcx_profile_dominant_kernel) is consumed by the kernel launch it asks
// for; an entry point that returns before that launch must not leave it armed.
struct ProfileRequestScope {
  ~ProfileRequestScope() { mcx::set_profile_events(nullptr, nullptr); }
};

struct ConvDims {
  int64_t B, Ci, Co, IH, IW, OH, OW, K, P;
};

// map_h x map_w is the spatial size of the sample map (output for convolution,
// input for transposed convolution).
int check_dims(const ConvDims &d, int64_t map_h, int64_t map_w, int dtype) {
  // samples are addressed with 32-bit byte offsets inside a plane
  const int64_t elem = dtype == MCX_F64 ? 8 : dtype == MCX_BF16 ? 2 : 4;
  if (d.IH * d.IW * elem > 0xffffffffLL || d.OH * d.OW * elem > 0xffffffffLL) return MCX_E_SHAPE;
  for (int64_t v : {d.B, d.Ci, d.Co, d.IH, d.IW, d.OH, d.OW, d.K, d.IH * d.IW, d.OH * d.OW})
    if (v <= 0 || v > 0x7fffffffLL) return MCX_E_SHAPE;
  if (d.P < 0 || d.P > 0x7fffffffLL || d.B > 65535) return MCX_E_SHAPE;
  // every plane and the whole map are addressed with 31-bit element offsets
  if (map_h * map_w * d.K * (d.P ? d.P : 1) * 2 > 0x7fffffffLL) return MCX_E_SHAPE;
  if (d.Ci * d.Co * d.K > 0x7fffffffLL) return MCX_E_SHAPE;
  return 0;
}

int check_ptrs(const void *a, const void *map, const void *iw, const void *w, int64_t P) {
  if (!a || !map || !w) return MCX_E_NULL;
  if ((P == 0) != (iw == nullptr)) return MCX_E_NULL;
  return 0;
}

size_t elem_size(int dtype) { return dtype == MCX_F64 ? 8 : dtype == MCX_BF16 ? 2 : 4; }
bool use_mfma(int dtype, int64_t P) {
  return (dtype == MCX_F32 || dtype == MCX_BF16) && mfma_supported(P);
}

template <typename T>
int fill_zero(T *p, int64_t n, hipStream_t s);
template <>
int fill_zero<float>(float *p, int64_t n, hipStream_t s) { return fill_f32(p, n, 0.f, s); }
template <>
int fill_zero<double>(double *p, int64_t n, hipStream_t s) { return fill_f64(p, n, 0.0, s); }

// ---- scratch sizes of the three operators -------------------------------------------
// SH x SW: the image sampled; MH x MW: the map
size_t gather_product_ws(int dtype, int64_t G, int64_t O, int64_t K, int64_t P, int64_t B,
                         int64_t SH, int64_t SW, int64_t MH, int64_t MW) {
  return use_mfma(dtype, P)
             ? mfma_gather_product_bytes(O, G, K, B, SH, SW, (int)elem_size(dtype), MH, MW)
             : 0;
}
size_t weight_grad_ws(int dtype, int64_t B, int64_t A, int64_t G, int64_t MH, int64_t MW,
                      int64_t K, int64_t P, int64_t GH, int64_t GW) {
  return use_mfma(dtype, P) ? mfma_weight_grad_bytes(B, A, G, MH, MW, K, GH, GW, elem_size(dtype)) : 0;
}
size_t product_scatter_ws(int dtype, int64_t B, int64_t S, int64_t D, int64_t K, int64_t P,
                          int64_t DH, int64_t DW, int64_t MH, int64_t MW) {
  return use_mfma(dtype, P)
             ? mfma_product_scatter_bytes(B, S, D, K, DH, DW, elem_size(dtype), MH, MW, P)
             : 0;
}
size_t bias_grad_ws(int dtype, int64_t B, int64_t C, int64_t N) {
  if (dtype == MCX_BF16) return mfma_bias_grad_bytes(B, C, N);
  return (channel_sum_scratch_bytes(B, C, N, elem_size(dtype)) + 255) & ~(size_t)255;
}

// ---- typed operators: scalar kernels for any T, matrix-core kernels for TD -----------
// y[b,o,n] = bias[o] + sum_{g,k} W[o,g,k] * sample(src[b,g], map[n,k]); n over MH x MW.
template <typename T>
int gather_product(bool mfma, const void *src, const void *map, const void *iw, const void *w,
                   const void *bias, void *y, void *ws, size_t ws_bytes, int64_t B, int64_t G,
                   int64_t O, int64_t SH, int64_t SW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                   int interp, hipStream_t s, const void *plan = nullptr);  // plan: see mcx.h

// dst[b,d] = bias[d] (or 0) + splat(sum_s W[s,d,k] * src[b,s,n], map[n,k]); n over MH x MW.
template <typename T>
int product_scatter(bool mfma, const void *src, const void *map, const void *iw, const void *w,
                    const void *bias, void *dst, void *ws, size_t ws_bytes, int64_t B, int64_t S,
                    int64_t D, int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                    int interp, hipStream_t s, const void *plan = nullptr);  // plan: see mcx.h

// gW[a,g,k] = sum_{b,n} plain[b,a,n] * sample(gath[b,g], map[n,k]); n over MH x MW.
template <typename T>
int weight_grad(bool mfma, const void *plain, const void *gath, const void *map, const void *iw,
                void *gw, void *ws, size_t ws_bytes, int64_t B, int64_t A, int64_t G, int64_t GH,
                int64_t GW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                hipStream_t s, void *plain_sum,  // plain_sum: matrix-core path only, may be NULL
                const void *plan = nullptr);

// gb[c] = sum over (b, n) of gy[b,c,n].
template <typename T>
int bias_grad(const void *gy, void *gb, void *ws, size_t ws_bytes, int64_t B, int64_t C, int64_t N,
              hipStream_t s);

#define MCX_SCALAR_OPS(T)                                                                          \
  template <>                                                                                      \
  int gather_product<T>(bool, const void *src, const void *map, const void *iw, const void *w,     \
                        const void *bias, void *y, void *, size_t, int64_t B, int64_t G,           \
                        int64_t O, int64_t SH, int64_t SW, int64_t MH, int64_t MW, int64_t K,      \
                        int64_t P, int interp, hipStream_t s, const void *) {                      \
    return generic_gather_product<T>((const T *)src, (const T *)map, (const T *)iw,                \
                                     (const T *)w, (const T *)bias, (T *)y, B, G, O, SH, SW,       \
                                     MH * MW, K, P, interp, s);                                    \
  }                                                                                                \
  template <>                                                                                      \
  int product_scatter<T>(bool, const void *src, const void *map, const void *iw, const void *w,    \
                         const void *bias, void *dst, void *, size_t, int64_t B, int64_t S,        \
                         int64_t D, int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,     \
                         int64_t P, int interp, hipStream_t s, const void *) {                     \
    int rc = bias ? fill_bias<T>((T *)dst, (const T *)bias, B, D, DH * DW, s)                      \
                  : fill_zero<T>((T *)dst, B * D * DH * DW, s);                                    \
    if (rc) return rc;                                                                             \
    return generic_product_scatter<T>((const T *)src, (const T *)map, (const T *)iw,               \
                                      (const T *)w, (T *)dst, B, S, D, DH, DW, MH * MW, K, P,      \
                                      interp, s);                                                  \
  }                                                                                                \
  template <>                                                                                      \
  int weight_grad<T>(bool, const void *plain, const void *gath, const void *map, const void *iw,   \
                     void *gw, void *, size_t, int64_t B, int64_t A, int64_t G, int64_t GH,        \
                     int64_t GW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,         \
                     hipStream_t s, void *, const void *) {                                        \
    return generic_weight_grad<T>((const T *)plain, (const T *)gath, (const T *)map,               \
                                  (const T *)iw, (T *)gw, B, A, G, GH, GW, MH * MW, K, P, interp,  \
                                  s);                                                              \
  }                                                                                                \
  template <>                                                                                      \
  int bias_grad<T>(const void *gy, void *gb, void *ws, size_t ws_bytes, int64_t B, int64_t C,      \
                   int64_t N, hipStream_t s) {                                                     \
    const size_t need = channel_sum_scratch_bytes(B, C, N, sizeof(T));                             \
    T *scratch = (ws && need > 0 && ws_bytes >= need) ? (T *)ws : nullptr;                         \
    return channel_sum<T>((const T *)gy, (T *)gb, scratch, B, C, N, s);                            \
  }

// double: scalar kernels only
MCX_SCALAR_OPS(double)

// float: matrix-core kernels when `mfma`, scalar kernels otherwise

template <>
int gather_product<float>(bool mfma, const void *src, const void *map, const void *iw,
                          const void *w, const void *bias, void *y, void *ws, size_t ws_bytes,
                          int64_t B, int64_t G, int64_t O, int64_t SH, int64_t SW, int64_t MH,
                          int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                          const void *plan) {
  if (!mfma)
    return generic_gather_product<float>((const float *)src, (const float *)map,
                                         (const float *)iw, (const float *)w, (const float *)bias,
                                         (float *)y, B, G, O, SH, SW, MH * MW, K, P, interp, s);
  if (!ws || ws_bytes < mfma_gather_product_bytes(O, G, K, B, SH, SW, 4, MH, MW))
    return MCX_E_WORKSPACE;
  return mfma_gather_product<float>((const float *)src, (const float *)map, (const float *)iw,
                                    (const float *)w, (const float *)bias, (float *)y, ws, B, G, O,
                                    SH, SW, MH, MW, K, P, interp, s, plan);
}

template <>
int product_scatter<float>(bool mfma, const void *src, const void *map, const void *iw,
                           const void *w, const void *bias, void *dst, void *ws, size_t ws_bytes,
                           int64_t B, int64_t S, int64_t D, int64_t DH, int64_t DW, int64_t MH,
                           int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                           const void *plan) {
  if (!mfma) {
    int rc = bias ? fill_bias<float>((float *)dst, (const float *)bias, B, D, DH * DW, s)
                  : fill_zero<float>((float *)dst, B * D * DH * DW, s);
    if (rc) return rc;
    return generic_product_scatter<float>((const float *)src, (const float *)map,
                                          (const float *)iw, (const float *)w, (float *)dst, B, S,
                                          D, DH, DW, MH * MW, K, P, interp, s);
  }
  if (!ws || ws_bytes < mfma_product_scatter_bytes(B, S, D, K, DH, DW, 4, MH, MW, P))
    return MCX_E_WORKSPACE;
  return mfma_product_scatter<float>((const float *)src, (const float *)map, (const float *)iw,
                                     (const float *)w, (const float *)bias, (float *)dst, ws, B, S,
                                     D, DH, DW, MH, MW, K, P, interp, s, plan);
}

template <>
int weight_grad<float>(bool mfma, const void *plain, const void *gath, const void *map,
                       const void *iw, void *gw, void *ws, size_t ws_bytes, int64_t B, int64_t A,
                       int64_t G, int64_t GH, int64_t GW, int64_t MH, int64_t MW, int64_t K,
                       int64_t P, int interp, hipStream_t s, void *plain_sum, const void *plan) {
  if (!mfma)
    return generic_weight_grad<float>((const float *)plain, (const float *)gath,
                                      (const float *)map, (const float *)iw, (float *)gw, B, A, G,
                                      GH, GW, MH * MW, K, P, interp, s);
  if (!ws || ws_bytes < mfma_weight_grad_bytes(B, A, G, MH, MW, K, GH, GW, 4))
    return MCX_E_WORKSPACE;
  return mfma_weight_grad<float>((const float *)plain, (const float *)gath, (const float *)map,
                                 (const float *)iw, (float *)gw, ws, B, A, G, GH, GW, MH, MW, K, P,
                                 interp, s, (float *)plain_sum, plan);
}

template <>
int bias_grad<float>(const void *gy, void *gb, void *ws, size_t ws_bytes, int64_t B, int64_t C,
                     int64_t N, hipStream_t s) {
  const size_t need = channel_sum_scratch_bytes(B, C, N, sizeof(float));
  float *scratch = (ws && need > 0 && ws_bytes >= need) ? (float *)ws : nullptr;
  return channel_sum<float>((const float *)gy, (float *)gb, scratch, B, C, N, s);
}

// bf16 storage: matrix-core kernels only (sample_map / interp_weights are fp32)
template <>
int gather_product<bf16_t>(bool mfma, const void *src, const void *map, const void *iw,
                           const void *w, const void *bias, void *y, void *ws, size_t ws_bytes,
                           int64_t B, int64_t G, int64_t O, int64_t SH, int64_t SW, int64_t MH,
                           int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                           const void *plan) {
  if (!mfma) return MCX_E_DTYPE;
  if (!ws || ws_bytes < mfma_gather_product_bytes(O, G, K, B, SH, SW, 2, MH, MW))
    return MCX_E_WORKSPACE;
  return mfma_gather_product<bf16_t>((const bf16_t *)src, (const float *)map, (const float *)iw,
                                     (const bf16_t *)w, (const bf16_t *)bias, (bf16_t *)y, ws, B,
                                     G, O, SH, SW, MH, MW, K, P, interp, s, plan);
}

template <>
int product_scatter<bf16_t>(bool mfma, const void *src, const void *map, const void *iw,
                            const void *w, const void *bias, void *dst, void *ws, size_t ws_bytes,
                            int64_t B, int64_t S, int64_t D, int64_t DH, int64_t DW, int64_t MH,
                            int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                            const void *plan) {
  if (!mfma) return MCX_E_DTYPE;
  if (!ws || ws_bytes < mfma_product_scatter_bytes(B, S, D, K, DH, DW, 2, MH, MW, P))
    return MCX_E_WORKSPACE;
  return mfma_product_scatter<bf16_t>((const bf16_t *)src, (const float *)map, (const float *)iw,
                                      (const bf16_t *)w, (const bf16_t *)bias, (bf16_t *)dst, ws,
                                      B, S, D, DH, DW, MH, MW, K, P, interp, s, plan);
}

template <>
int weight_grad<bf16_t>(bool mfma, const void *plain, const void *gath, const void *map,
                        const void *iw, void *gw, void *ws, size_t ws_bytes, int64_t B, int64_t A,
                        int64_t G, int64_t GH, int64_t GW, int64_t MH, int64_t MW, int64_t K,
                        int64_t P, int interp, hipStream_t s, void *plain_sum,
                        const void *plan) {
  if (!mfma) return MCX_E_DTYPE;
  if (!ws || ws_bytes < mfma_weight_grad_bytes(B, A, G, MH, MW, K, GH, GW, 2))
    return MCX_E_WORKSPACE;
  return mfma_weight_grad<bf16_t>((const bf16_t *)plain, (const bf16_t *)gath, (const float *)map,
                                  (const float *)iw, (bf16_t *)gw, ws, B, A, G, GH, GW, MH, MW, K,
                                  P, interp, s, (bf16_t *)plain_sum, plan);
}

template <>
int bias_grad<bf16_t>(const void *gy, void *gb, void *ws, size_t ws_bytes, int64_t B, int64_t C,
                      int64_t N, hipStream_t s) {
  if (!ws || ws_bytes < mfma_bias_grad_bytes(B, C, N)) return MCX_E_WORKSPACE;
  return mfma_bias_grad<bf16_t>((const bf16_t *)gy, (bf16_t *)gb, ws, B, C, N, s);
}

// ---- the four layer-level operations, in terms of the operators ----------------------
template <typename T>
int conv_forward_t(bool mfma, const void *x, const void *map, const void *iw, const void *w,
                   const void *bias, void *y, void *ws, size_t ws_bytes, const ConvDims &d,
                   int interp, hipStream_t s, const void *plan = nullptr) {
  return gather_product<T>(mfma, x, map, iw, w, bias, y, ws, ws_bytes, d.B, d.Ci, d.Co, d.IH, d.IW,
                           d.OH, d.OW, d.K, d.P, interp, s, plan);
}

template <typename T>
int conv_backward_t(bool mfma, const void *gy, const void *map, const void *iw, const void *x,
                    const void *w, void *gx, void *gw, void *gb, void *ws, size_t ws_bytes,
                    const ConvDims &d, int interp, hipStream_t s, const void *plan = nullptr) {
  int rc = 0;
  if (gx && (rc = product_scatter<T>(mfma, gy, map, iw, w, nullptr, gx, ws, ws_bytes, d.B, d.Co,
                                     d.Ci, d.IH, d.IW, d.OH, d.OW, d.K, d.P, interp, s, plan)))
    return rc;
  // the matrix-core weight gradient stages every tile of gy: it sums them for the bias
  // gradient on the way
  const bool fused_bias = gw && gb && mfma;
  if (gw && (rc = weight_grad<T>(mfma, gy, x, map, iw, gw, ws, ws_bytes, d.B, d.Co, d.Ci, d.IH,
                                 d.IW, d.OH, d.OW, d.K, d.P, interp, s, fused_bias ? gb : nullptr,
                                 plan)))
    return rc;
  if (gb && !fused_bias) rc = bias_grad<T>(gy, gb, ws, ws_bytes, d.B, d.Co, d.OH * d.OW, s);
  return rc;
}

template <typename T>
int tconv_forward_t(bool mfma, const void *x, const void *map, const void *iw, const void *w,
                    const void *bias, void *y, void *ws, size_t ws_bytes, const ConvDims &d,
                    int interp, hipStream_t s, const void *plan = nullptr) {
  return product_scatter<T>(mfma, x, map, iw, w, bias, y, ws, ws_bytes, d.B, d.Ci, d.Co, d.OH,
                            d.OW, d.IH, d.IW, d.K, d.P, interp, s, plan);
}

template <typename T>
int tconv_backward_t(bool mfma, const void *gy, const void *map, const void *iw, const void *x,
                     const void *w, void *gx, void *gw, void *gb, void *ws, size_t ws_bytes,
                     const ConvDims &d, int interp, hipStream_t s, const void *plan = nullptr) {
  int rc = 0;
  // grad_input[b,ci] = sum_{co,k} W[ci,co,k] * sample(gy[b,co], map[n,k])
  if (gx && (rc = gather_product<T>(mfma, gy, map, iw, w, nullptr, gx, ws, ws_bytes, d.B, d.Co,
                                    d.Ci, d.OH, d.OW, d.IH, d.IW, d.K, d.P, interp, s, plan)))
    return rc;
  if (gw && (rc = weight_grad<T>(mfma, x, gy, map, iw, gw, ws, ws_bytes, d.B, d.Ci, d.Co, d.OH,
                                 d.OW, d.IH, d.IW, d.K, d.P, interp, s, nullptr, plan)))
    return rc;
  if (gb) rc = bias_grad<T>(gy, gb, ws, ws_bytes, d.B, d.Co, d.OH * d.OW, s);
  return rc;
}

#define MCX_DISPATCH_DTYPE(dtype, CALL)           \
  switch (dtype) {                                \
    case MCX_F32: { using T = float; return CALL; }   \
    case MCX_F64: { using T = double; return CALL; }  \
    case MCX_BF16: { using T = bf16_t; return CALL; } \
    default: return MCX_E_DTYPE;                  \
  }

}  // namespace

extern "C" size_t mcx_conv_forward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                             int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                             int64_t P, int dtype) {
  return gather_product_ws(dtype, Ci, Co, K, P, B, IH, IW, OH, OW);
}

extern "C" int mcx_conv_forward(const void *x, const void *map, const void *iw, const void *w,
                                const void *bias, void *y, void *workspace,
                                size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                int64_t P, int interp, int dtype, void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW, dtype)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  MCX_DISPATCH_DTYPE(dtype, conv_forward_t<T>(mfma, x, map, iw, w, bias, y, workspace,
                                              workspace_bytes, d, interp, s));
}

extern "C" int mcx_conv_forward_static(const void *x, const void *map, const void *iw,
                                       const void *w, const void *bias, void *y, int64_t B,
                                       int64_t Ci, int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                                       int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                       void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW, dtype)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  if (dtype != MCX_F32 && dtype != MCX_F64 && dtype != MCX_BF16) return MCX_E_DTYPE;
  const size_t need = gather_product_ws(dtype, Ci, Co, K, P, B, IH, IW, OH, OW);
  if (need > kStaticScratchBytes) return MCX_E_STATIC_LIMIT;
  int rc = 0;
  void *ws = static_scratch_of_current_device(&rc);
  if (!ws) return rc;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  // the kernels overwrite every word of the scratch they read (the weight-packing kernel
  // clears the flag word beside the packed weights), so nothing of the last call survives
  MCX_DISPATCH_DTYPE(dtype, conv_forward_t<T>(mfma, x, map, iw, w, bias, y, ws,
                                              kStaticScratchBytes, d, interp, s));
}

extern "C" size_t mcx_conv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                              int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                              int64_t P, int dtype) {
  // the gradients run one after the other on the stream and share the scratch
  return std::max({weight_grad_ws(dtype, B, Co, Ci, OH, OW, K, P, IH, IW),
                   product_scatter_ws(dtype, B, Co, Ci, K, P, IH, IW, OH, OW),
                   bias_grad_ws(dtype, B, Co, OH * OW)});
}

extern "C" int mcx_conv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                 const void *w, void *gx, void *gw, void *gb, void *workspace,
                                 size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW, dtype)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  MCX_DISPATCH_DTYPE(dtype, conv_backward_t<T>(mfma, gy, map, iw, x, w, gx, gw, gb, workspace,
                                               workspace_bytes, d, interp, s));
}

extern "C" size_t mcx_conv_plan_bytes(int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                      int64_t P, int dtype) {
  if (IH <= 0 || IW <= 0 || OH <= 0 || OW <= 0 || K <= 0 || P < 0) return 0;
  return use_mfma(dtype, P) ? mfma_scatter_plan_bytes(IH, IW, OH, OW, K, P) : 0;
}

extern "C" int mcx_conv_plan_build(const void *map, const void *iw, void *plan, size_t plan_bytes,
                                   mcx_plan_desc *desc, int64_t IH, int64_t IW, int64_t OH,
                                   int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                   void *stream) {
  if (IH <= 0 || IW <= 0 || OH <= 0 || OW <= 0 || K <= 0 || P < 0) return MCX_E_SHAPE;
  if (!map || !plan || !desc || (P > 0) != (iw != nullptr)) return MCX_E_NULL;
  if (!use_mfma(dtype, P)) return MCX_E_DTYPE;
  const size_t need = mfma_scatter_plan_bytes(IH, IW, OH, OW, K, P);
  if (need == 0) return MCX_E_SHAPE;
  if (plan_bytes < need) return MCX_E_WORKSPACE;
  desc->magic = 0;  // (not a plan until the build has been enqueued)
  if (int rc = mfma_scatter_plan_build((const float *)map, (const float *)iw, plan, IH, IW, OH, OW,
                                       K, P, interp, (hipStream_t)stream))
    return rc;
  // (the plan holds element indices and fp32 weights: the same for fp32 and bf16 data)
  plan_desc_fill(desc, MCX_PLAN_CONV, interp, MCX_F32, IH, IW, OH, OW, K, P, plan, need, map, iw);
  return 0;
}

namespace {
// A plan, when given, must be the one mcx_conv_plan_build made at this address for this map,
// interpolation and these sizes (SH x SW: the image the map samples; MH x MW: the map).
int check_plan(const void *plan, size_t plan_bytes, const mcx_plan_desc *desc, bool mfma,
               int64_t SH, int64_t SW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
               const void *map, const void *iw) {
  if (!plan) return 0;
  if (!mfma) return MCX_E_DTYPE;
  const size_t need = mfma_scatter_plan_bytes(SH, SW, MH, MW, K, P);
  if (need == 0 || plan_bytes < need) return MCX_E_WORKSPACE;
  return plan_desc_check(desc, MCX_PLAN_CONV, interp, MCX_F32, SH, SW, MH, MW, K, P, plan,
                         plan_bytes, true, map, iw);
}
}  // namespace

extern "C" int mcx_conv_backward_planned(const void *gy, const void *map, const void *iw,
                                         const void *x, const void *w, void *gx, void *gw,
                                         void *gb, void *workspace, size_t workspace_bytes,
                                         const void *plan, size_t plan_bytes,
                                         const mcx_plan_desc *desc, int64_t B, int64_t Ci,
                                         int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                                         int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                         void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW, dtype)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  if (int rc = check_plan(plan, plan_bytes, desc, mfma, IH, IW, OH, OW, K, P, interp, map, iw))
    return rc;
  MCX_DISPATCH_DTYPE(dtype, conv_backward_t<T>(mfma, gy, map, iw, x, w, gx, gw, gb, workspace,
                                               workspace_bytes, d, interp, s, plan));
}

extern "C" int mcx_conv_forward_planned(const void *x, const void *map, const void *iw,
                                        const void *w, const void *bias, void *y, void *workspace,
                                        size_t workspace_bytes, const void *plan,
                                        size_t plan_bytes, const mcx_plan_desc *desc, int64_t B,
                                        int64_t Ci, int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                                        int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                        void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW, dtype)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  if (int rc = check_plan(plan, plan_bytes, desc, mfma, IH, IW, OH, OW, K, P, interp, map, iw))
    return rc;
  MCX_DISPATCH_DTYPE(dtype, conv_forward_t<T>(mfma, x, map, iw, w, bias, y, workspace,
                                              workspace_bytes, d, interp, s, plan));
}

extern "C" int mcx_tconv_forward_planned(const void *x, const void *map, const void *iw,
                                         const void *w, const void *bias, void *y,
                                         void *workspace, size_t workspace_bytes, const void *plan,
                                         size_t plan_bytes, const mcx_plan_desc *desc, int64_t B,
                                         int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                                         int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                                         int dtype, void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW, dtype)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  if (int rc = check_plan(plan, plan_bytes, desc, mfma, OH, OW, IH, IW, K, P, interp, map, iw))
    return rc;
  MCX_DISPATCH_DTYPE(dtype, tconv_forward_t<T>(mfma, x, map, iw, w, bias, y, workspace,
                                               workspace_bytes, d, interp, s, plan));
}

extern "C" int mcx_tconv_backward_planned(const void *gy, const void *map, const void *iw,
                                          const void *x, const void *w, void *gx, void *gw,
                                          void *gb, void *workspace, size_t workspace_bytes,
                                          const void *plan, size_t plan_bytes,
                                          const mcx_plan_desc *desc, int64_t B, int64_t Ci,
                                          int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                                          int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                                          void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW, dtype)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  if (int rc = check_plan(plan, plan_bytes, desc, mfma, OH, OW, IH, IW, K, P, interp, map, iw))
    return rc;
  MCX_DISPATCH_DTYPE(dtype, tconv_backward_t<T>(mfma, gy, map, iw, x, w, gx, gw, gb, workspace,
                                                workspace_bytes, d, interp, s, plan));
}

extern "C" size_t mcx_tconv_forward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                              int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                              int64_t P, int dtype) {
  return product_scatter_ws(dtype, B, Ci, Co, K, P, OH, OW, IH, IW);
}

extern "C" int mcx_tconv_forward(const void *x, const void *map, const void *iw, const void *w,
                                 const void *bias, void *y, void *workspace,
                                 size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW, dtype)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  MCX_DISPATCH_DTYPE(dtype, tconv_forward_t<T>(mfma, x, map, iw, w, bias, y, workspace,
                                               workspace_bytes, d, interp, s));
}

extern "C" size_t mcx_tconv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                               int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                               int64_t P, int dtype) {
  // backward-input is a gather-product with the channel roles swapped; the
  // gradients run one after the other and share the scratch
  return std::max({gather_product_ws(dtype, Co, Ci, K, P, B, OH, OW, IH, IW),
                   weight_grad_ws(dtype, B, Ci, Co, IH, IW, K, P, OH, OW),
                   bias_grad_ws(dtype, B, Co, OH * OW)});
}

extern "C" int mcx_tconv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                  const void *w, void *gx, void *gw, void *gb, void *workspace,
                                  size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                  int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                  int64_t P, int interp, int dtype, void *stream) {
  ProfileRequestScope profile_scope;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW, dtype)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  const bool mfma = use_mfma(dtype, P);
  MCX_DISPATCH_DTYPE(dtype, tconv_backward_t<T>(mfma, gy, map, iw, x, w, gx, gw, gb, workspace,
                                                workspace_bytes, d, interp, s));
}

extern "C" int mcx_abi_version(void) { return 11; }

extern "C" int mcx_profile_dominant_kernel(void *start_event, void *stop_event) {
  mcx::set_profile_events(start_event, stop_event);
  return MCX_OK;
}

extern "C" const char *mcx_error_string(int code) {
  switch (code) {
    case MCX_OK: return "success";
    case MCX_E_DTYPE: return "mcx: dtype (or dtype / interpolation-point combination) not supported by this entry point";
    case MCX_E_SHAPE: return "mcx: invalid or too large dimension";
    case MCX_E_NULL: return "mcx: required pointer is NULL, or interp_weights and P disagree";
    case MCX_E_WORKSPACE: return "mcx: workspace missing or too small";
    case MCX_E_PLAN:
      return "mcx: this plan was not built for this operation, map, interpolation or size "
             "(or its descriptor is missing or damaged)";
    case MCX_E_STATIC_LIMIT:
      return "mcx: this problem needs more scratch than the library's static buffer holds; "
             "use the entry point that takes a workspace";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "mcx: unknown error";
  }
}
