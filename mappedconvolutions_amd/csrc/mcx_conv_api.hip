// extern "C" entry points of the mapped (transposed) convolution.  Validates the
// arguments, then routes each of the three products (gather-product,
// product-scatter, weight gradient; see mcx_conv_generic.hip for the roles) to the
// matrix-core kernels when they cover the case and to the scalar kernels otherwise.
#include <algorithm>
#include <initializer_list>

#include "mcx.h"
#include "mcx_conv.h"

using namespace mcx;

namespace {

struct ConvDims {
  int64_t B, Ci, Co, IH, IW, OH, OW, K, P;
};

// map_h x map_w is the spatial size of the sample map (output for convolution,
// input for transposed convolution).
int check_dims(const ConvDims &d, int64_t map_h, int64_t map_w) {
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

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

template <typename T>
int fill_zero(T *p, int64_t n, hipStream_t s);
template <>
int fill_zero<float>(float *p, int64_t n, hipStream_t s) { return fill_f32(p, n, 0.f, s); }
template <>
int fill_zero<double>(double *p, int64_t n, hipStream_t s) { return fill_f64(p, n, 0.0, s); }

// ---- the three operators, typed ------------------------------------------------

// y[b,o,n] = bias[o] + sum_{g,k} W[o,g,k] * sample(src[b,g], map[n,k]); n over MH x MW.
size_t gather_product_ws(int dtype, int64_t G, int64_t O, int64_t K, int64_t P) {
  if (dtype == MCX_F32 && mfma_f32_gather_product_supported(P))
    return align256(mfma_f32_packed_weight_bytes(O, G, K));
  return 0;
}

template <typename T>
int gather_product(const T *src, const T *map, const T *iw, const T *w, const T *bias, T *y,
                   void *ws, size_t ws_bytes, int64_t B, int64_t G, int64_t O, int64_t SH,
                   int64_t SW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                   hipStream_t s) {
  (void)ws;
  (void)ws_bytes;
  return generic_gather_product<T>(src, map, iw, w, bias, y, B, G, O, SH, SW, MH * MW, K, P,
                                   interp, s);
}

template <>
int gather_product<float>(const float *src, const float *map, const float *iw, const float *w,
                          const float *bias, float *y, void *ws, size_t ws_bytes, int64_t B,
                          int64_t G, int64_t O, int64_t SH, int64_t SW, int64_t MH, int64_t MW,
                          int64_t K, int64_t P, int interp, hipStream_t s) {
  if (!mfma_f32_gather_product_supported(P))
    return generic_gather_product<float>(src, map, iw, w, bias, y, B, G, O, SH, SW, MH * MW, K, P,
                                         interp, s);
  if (!ws || ws_bytes < gather_product_ws(MCX_F32, G, O, K, P)) return MCX_E_WORKSPACE;
  return mfma_f32_gather_product(src, map, iw, w, bias, y, (float *)ws, B, G, O, SH, SW, MH, MW,
                                 K, P, interp, s);
}

// gW[a,g,k] = sum_{b,n} plain[b,a,n] * sample(gath[b,g], map[n,k]); n over MH x MW.
size_t weight_grad_ws(int dtype, int64_t B, int64_t A, int64_t G, int64_t MH, int64_t MW,
                      int64_t K, int64_t P) {
  if (dtype == MCX_F32 && mfma_f32_weight_grad_supported(P))
    return align256(mfma_f32_weight_grad_bytes(B, A, G, MH, MW, K));
  return 0;
}

template <typename T>
int weight_grad(const T *plain, const T *gath, const T *map, const T *iw, T *gw, void *ws,
                size_t ws_bytes, int64_t B, int64_t A, int64_t G, int64_t GH, int64_t GW,
                int64_t MH, int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s) {
  (void)ws;
  (void)ws_bytes;
  return generic_weight_grad<T>(plain, gath, map, iw, gw, B, A, G, GH, GW, MH * MW, K, P, interp,
                                s);
}

template <>
int weight_grad<float>(const float *plain, const float *gath, const float *map, const float *iw,
                       float *gw, void *ws, size_t ws_bytes, int64_t B, int64_t A, int64_t G,
                       int64_t GH, int64_t GW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                       int interp, hipStream_t s) {
  if (!mfma_f32_weight_grad_supported(P))
    return generic_weight_grad<float>(plain, gath, map, iw, gw, B, A, G, GH, GW, MH * MW, K, P,
                                      interp, s);
  if (!ws || ws_bytes < weight_grad_ws(MCX_F32, B, A, G, MH, MW, K, P)) return MCX_E_WORKSPACE;
  return mfma_f32_weight_grad(plain, gath, map, iw, gw, (float *)ws, B, A, G, GH, GW, MH, MW, K,
                              P, interp, s);
}

// dst[b,d] += splat(sum_s W[s,d,k] * src[b,s,n], map[n,k]); n over MH x MW; dst pre-initialised.
size_t product_scatter_ws(int dtype, int64_t S, int64_t D, int64_t K, int64_t P, int64_t DH,
                          int64_t DW) {
  if (dtype == MCX_F32 && mfma_f32_product_scatter_supported(P))
    return align256(mfma_f32_product_scatter_bytes(S, D, K, DH, DW));
  return 0;
}

// `bias` (may be NULL) is the per-channel value dst was initialised with.
template <typename T>
int product_scatter(const T *src, const T *map, const T *iw, const T *w, const T *bias, T *dst,
                    void *ws, size_t ws_bytes, int64_t B, int64_t S, int64_t D, int64_t DH,
                    int64_t DW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                    hipStream_t s) {
  (void)ws;
  (void)ws_bytes;
  (void)bias;
  return generic_product_scatter<T>(src, map, iw, w, dst, B, S, D, DH, DW, MH * MW, K, P, interp,
                                    s);
}

template <>
int product_scatter<float>(const float *src, const float *map, const float *iw, const float *w,
                           const float *bias, float *dst, void *ws, size_t ws_bytes, int64_t B,
                           int64_t S, int64_t D, int64_t DH, int64_t DW, int64_t MH, int64_t MW,
                           int64_t K, int64_t P, int interp, hipStream_t s) {
  if (!mfma_f32_product_scatter_supported(P))
    return generic_product_scatter<float>(src, map, iw, w, dst, B, S, D, DH, DW, MH * MW, K, P,
                                          interp, s);
  if (!ws || ws_bytes < product_scatter_ws(MCX_F32, S, D, K, P, DH, DW)) return MCX_E_WORKSPACE;
  return mfma_f32_product_scatter(src, map, iw, w, bias, dst, ws, B, S, D, DH, DW, MH, MW, K, P,
                                  interp, s);
}

// gb[c] = sum over (b, n) of gy[b,c,n]; uses the scratch when it is large enough.
template <typename T>
int bias_grad(const T *gy, T *gb, void *ws, size_t ws_bytes, int64_t B, int64_t C, int64_t N,
              hipStream_t s) {
  const size_t need = channel_sum_scratch_bytes(B, C, N, sizeof(T));
  T *scratch = (ws && need > 0 && ws_bytes >= need) ? (T *)ws : nullptr;
  return channel_sum<T>(gy, gb, scratch, B, C, N, s);
}

template <typename T>
int conv_forward_t(const void *x, const void *map, const void *iw, const void *w, const void *bias,
                   void *y, void *ws, size_t ws_bytes, const ConvDims &d, int interp,
                   hipStream_t s) {
  return gather_product<T>((const T *)x, (const T *)map, (const T *)iw, (const T *)w,
                           (const T *)bias, (T *)y, ws, ws_bytes, d.B, d.Ci, d.Co, d.IH, d.IW,
                           d.OH, d.OW, d.K, d.P, interp, s);
}

template <typename T>
int conv_backward_t(const void *gy, const void *map, const void *iw, const void *x, const void *w,
                    void *gx, void *gw, void *gb, void *ws, size_t ws_bytes, const ConvDims &d,
                    int interp, hipStream_t s) {
  int rc = 0;
  const int64_t N = d.OH * d.OW;
  (void)N;
  if (gx) {
    if ((rc = fill_zero<T>((T *)gx, d.B * d.Ci * d.IH * d.IW, s))) return rc;
    if ((rc = product_scatter<T>((const T *)gy, (const T *)map, (const T *)iw, (const T *)w,
                                 (const T *)nullptr, (T *)gx, ws, ws_bytes, d.B, d.Co, d.Ci, d.IH,
                                 d.IW, d.OH, d.OW, d.K, d.P, interp, s)))
      return rc;
  }
  if (gw) {
    if ((rc = weight_grad<T>((const T *)gy, (const T *)x, (const T *)map, (const T *)iw, (T *)gw,
                             ws, ws_bytes, d.B, d.Co, d.Ci, d.IH, d.IW, d.OH, d.OW, d.K, d.P,
                             interp, s)))
      return rc;
  }
  if (gb) rc = bias_grad<T>((const T *)gy, (T *)gb, ws, ws_bytes, d.B, d.Co, d.OH * d.OW, s);
  return rc;
}

template <typename T>
int tconv_forward_t(const void *x, const void *map, const void *iw, const void *w,
                    const void *bias, void *y, void *ws, size_t ws_bytes, const ConvDims &d,
                    int interp, hipStream_t s) {
  int rc = fill_bias<T>((T *)y, (const T *)bias, d.B, d.Co, d.OH * d.OW, s);
  if (rc) return rc;
  return product_scatter<T>((const T *)x, (const T *)map, (const T *)iw, (const T *)w,
                            (const T *)bias, (T *)y, ws, ws_bytes, d.B, d.Ci, d.Co, d.OH, d.OW,
                            d.IH, d.IW, d.K, d.P, interp, s);
}

template <typename T>
int tconv_backward_t(const void *gy, const void *map, const void *iw, const void *x,
                     const void *w, void *gx, void *gw, void *gb, void *ws, size_t ws_bytes,
                     const ConvDims &d, int interp, hipStream_t s) {
  int rc = 0;
  const int64_t N = d.IH * d.IW;
  if (gx) {
    // grad_input[b,ci] = sum_{co,k} W[ci,co,k] * sample(gy[b,co], map[n,k])
    if ((rc = gather_product<T>((const T *)gy, (const T *)map, (const T *)iw, (const T *)w,
                                (const T *)nullptr, (T *)gx, ws, ws_bytes, d.B, d.Co, d.Ci, d.OH,
                                d.OW, d.IH, d.IW, d.K, d.P, interp, s)))
      return rc;
  }
  if (gw) {
    if ((rc = weight_grad<T>((const T *)x, (const T *)gy, (const T *)map, (const T *)iw, (T *)gw,
                             ws, ws_bytes, d.B, d.Ci, d.Co, d.OH, d.OW, d.IH, d.IW, d.K, d.P,
                             interp, s)))
      return rc;
  }
  if (gb) rc = bias_grad<T>((const T *)gy, (T *)gb, ws, ws_bytes, d.B, d.Co, d.OH * d.OW, s);
  return rc;
}

}  // namespace

extern "C" size_t mcx_conv_forward_workspace(int64_t, int64_t Ci, int64_t Co, int64_t, int64_t,
                                             int64_t, int64_t, int64_t K, int64_t P, int dtype) {
  return gather_product_ws(dtype, Ci, Co, K, P);
}

extern "C" int mcx_conv_forward(const void *x, const void *map, const void *iw, const void *w,
                                const void *bias, void *y, void *workspace,
                                size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32:
      return conv_forward_t<float>(x, map, iw, w, bias, y, workspace, workspace_bytes, d, interp, s);
    case MCX_F64:
      return conv_forward_t<double>(x, map, iw, w, bias, y, workspace, workspace_bytes, d, interp,
                                    s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" size_t mcx_conv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                              int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                              int64_t P, int dtype) {
  // the gradients run one after the other on the stream and share the scratch
  const size_t elem = dtype == MCX_F64 ? 8 : 4;
  return std::max({weight_grad_ws(dtype, B, Co, Ci, OH, OW, K, P),
                   product_scatter_ws(dtype, Co, Ci, K, P, IH, IW),
                   align256(channel_sum_scratch_bytes(B, Co, OH * OW, elem))});
}

extern "C" int mcx_conv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                 const void *w, void *gx, void *gw, void *gb, void *workspace,
                                 size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, OH, OW)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32:
      return conv_backward_t<float>(gy, map, iw, x, w, gx, gw, gb, workspace, workspace_bytes, d,
                                    interp, s);
    case MCX_F64:
      return conv_backward_t<double>(gy, map, iw, x, w, gx, gw, gb, workspace, workspace_bytes, d,
                                     interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" size_t mcx_tconv_forward_workspace(int64_t, int64_t Ci, int64_t Co, int64_t, int64_t,
                                              int64_t OH, int64_t OW, int64_t K, int64_t P,
                                              int dtype) {
  return product_scatter_ws(dtype, Ci, Co, K, P, OH, OW);
}

extern "C" int mcx_tconv_forward(const void *x, const void *map, const void *iw, const void *w,
                                 const void *bias, void *y, void *workspace,
                                 size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32:
      return tconv_forward_t<float>(x, map, iw, w, bias, y, workspace, workspace_bytes, d, interp,
                                    s);
    case MCX_F64:
      return tconv_forward_t<double>(x, map, iw, w, bias, y, workspace, workspace_bytes, d,
                                     interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" size_t mcx_tconv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                                               int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                               int64_t P, int dtype) {
  // backward-input is a gather-product with the channel roles swapped; the
  // gradients run one after the other and share the scratch
  const size_t elem = dtype == MCX_F64 ? 8 : 4;
  return std::max({gather_product_ws(dtype, Co, Ci, K, P),
                   weight_grad_ws(dtype, B, Ci, Co, IH, IW, K, P),
                   align256(channel_sum_scratch_bytes(B, Co, OH * OW, elem))});
}

extern "C" int mcx_tconv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                  const void *w, void *gx, void *gw, void *gb, void *workspace,
                                  size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                  int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                  int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d, IH, IW)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32:
      return tconv_backward_t<float>(gy, map, iw, x, w, gx, gw, gb, workspace, workspace_bytes, d,
                                     interp, s);
    case MCX_F64:
      return tconv_backward_t<double>(gy, map, iw, x, w, gx, gw, gb, workspace, workspace_bytes, d,
                                      interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" int mcx_abi_version(void) { return 2; }

extern "C" const char *mcx_error_string(int code) {
  switch (code) {
    case MCX_OK: return "success";
    case MCX_E_DTYPE: return "mcx: dtype not supported by this entry point";
    case MCX_E_SHAPE: return "mcx: invalid or too large dimension";
    case MCX_E_NULL: return "mcx: required pointer is NULL, or interp_weights and P disagree";
    case MCX_E_WORKSPACE: return "mcx: workspace missing or too small";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "mcx: unknown error";
  }
}
