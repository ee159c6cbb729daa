// extern "C" entry points of the mapped (transposed) convolution.  Validates the
// arguments, then routes each of the three products to a kernel family.
#include <initializer_list>

#include "mcx.h"
#include "mcx_conv.h"

using namespace mcx;

namespace {

struct ConvDims {
  int64_t B, Ci, Co, IH, IW, OH, OW, K, P;
};

int check_dims(const ConvDims &d) {
  for (int64_t v : {d.B, d.Ci, d.Co, d.IH, d.IW, d.OH, d.OW, d.K, d.IH * d.IW, d.OH * d.OW})
    if (v <= 0 || v > 0x7fffffffLL) return MCX_E_SHAPE;
  if (d.P < 0 || d.P > 0x7fffffffLL || d.B > 65535) return MCX_E_SHAPE;
  const int64_t pm = d.P ? d.P : 1;
  // Largest tensors must be addressable with 63-bit element offsets and each
  // plane / map with 31-bit ones.
  if (d.OH * d.OW * d.K * pm * 2 > 0x7fffffffLL && d.IH * d.IW * d.K * pm * 2 > 0x7fffffffLL)
    return MCX_E_SHAPE;
  return 0;
}

template <typename T>
int conv_forward_t(const void *x, const void *map, const void *iw, const void *w, const void *bias,
                   void *y, const ConvDims &d, int interp, hipStream_t s) {
  return generic_gather_product<T>((const T *)x, (const T *)map, (const T *)iw, (const T *)w,
                                   (const T *)bias, (T *)y, d.B, d.Ci, d.Co, d.IH, d.IW,
                                   d.OH * d.OW, d.K, d.P, interp, s);
}

template <typename T>
int fill_zero(T *p, int64_t n, hipStream_t s);
template <>
int fill_zero<float>(float *p, int64_t n, hipStream_t s) { return fill_f32(p, n, 0.f, s); }
template <>
int fill_zero<double>(double *p, int64_t n, hipStream_t s) { return fill_f64(p, n, 0.0, s); }

template <typename T>
int conv_backward_t(const void *gy, const void *map, const void *iw, const void *x, const void *w,
                    void *gx, void *gw, void *gb, const ConvDims &d, int interp, hipStream_t s) {
  int rc = 0;
  const int64_t N = d.OH * d.OW;
  if (gx) {
    if ((rc = fill_zero<T>((T *)gx, d.B * d.Ci * d.IH * d.IW, s))) return rc;
    if ((rc = generic_product_scatter<T>((const T *)gy, (const T *)map, (const T *)iw,
                                         (const T *)w, (T *)gx, d.B, d.Co, d.Ci, d.IH, d.IW, N,
                                         d.K, d.P, interp, s)))
      return rc;
  }
  if (gw) {
    if ((rc = generic_weight_grad<T>((const T *)gy, (const T *)x, (const T *)map, (const T *)iw,
                                     (T *)gw, d.B, d.Co, d.Ci, d.IH, d.IW, N, d.K, d.P, interp,
                                     s)))
      return rc;
  }
  if (gb) rc = channel_sum<T>((const T *)gy, (T *)gb, d.B, d.Co, N, s);
  return rc;
}

template <typename T>
int tconv_forward_t(const void *x, const void *map, const void *iw, const void *w,
                    const void *bias, void *y, const ConvDims &d, int interp, hipStream_t s) {
  int rc = fill_bias<T>((T *)y, (const T *)bias, d.B, d.Co, d.OH * d.OW, s);
  if (rc) return rc;
  return generic_product_scatter<T>((const T *)x, (const T *)map, (const T *)iw, (const T *)w,
                                    (T *)y, d.B, d.Ci, d.Co, d.OH, d.OW, d.IH * d.IW, d.K, d.P,
                                    interp, s);
}

template <typename T>
int tconv_backward_t(const void *gy, const void *map, const void *iw, const void *x,
                     const void *w, void *gx, void *gw, void *gb, const ConvDims &d, int interp,
                     hipStream_t s) {
  int rc = 0;
  const int64_t N = d.IH * d.IW;
  if (gx) {
    if ((rc = generic_gather_product<T>((const T *)gy, (const T *)map, (const T *)iw,
                                        (const T *)w, (const T *)nullptr, (T *)gx, d.B, d.Co,
                                        d.Ci, d.OH, d.OW, N, d.K, d.P, interp, s)))
      return rc;
  }
  if (gw) {
    if ((rc = generic_weight_grad<T>((const T *)x, (const T *)gy, (const T *)map, (const T *)iw,
                                     (T *)gw, d.B, d.Ci, d.Co, d.OH, d.OW, N, d.K, d.P, interp,
                                     s)))
      return rc;
  }
  if (gb) rc = channel_sum<T>((const T *)gy, (T *)gb, d.B, d.Co, d.OH * d.OW, s);
  return rc;
}

int check_ptrs(const void *a, const void *map, const void *iw, const void *w, int64_t P) {
  if (!a || !map || !w) return MCX_E_NULL;
  if ((P == 0) != (iw == nullptr)) return MCX_E_NULL;
  return 0;
}

}  // namespace

extern "C" int mcx_conv_forward(const void *x, const void *map, const void *iw, const void *w,
                                const void *bias, void *y, int64_t B, int64_t Ci, int64_t Co,
                                int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32: return conv_forward_t<float>(x, map, iw, w, bias, y, d, interp, s);
    case MCX_F64: return conv_forward_t<double>(x, map, iw, w, bias, y, d, interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" size_t mcx_conv_backward_workspace(int64_t, int64_t, int64_t, int64_t, int64_t,
                                              int64_t, int64_t, int64_t, int64_t, int) {
  return 0;
}

extern "C" int mcx_conv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                 const void *w, void *gx, void *gw, void *gb, void *workspace,
                                 size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  (void)workspace;
  (void)workspace_bytes;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32: return conv_backward_t<float>(gy, map, iw, x, w, gx, gw, gb, d, interp, s);
    case MCX_F64: return conv_backward_t<double>(gy, map, iw, x, w, gx, gw, gb, d, interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" int mcx_tconv_forward(const void *x, const void *map, const void *iw, const void *w,
                                 const void *bias, void *y, int64_t B, int64_t Ci, int64_t Co,
                                 int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                 int64_t P, int interp, int dtype, void *stream) {
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d)) return rc;
  if (int rc = check_ptrs(x, map, iw, w, P)) return rc;
  if (!bias || !y) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32: return tconv_forward_t<float>(x, map, iw, w, bias, y, d, interp, s);
    case MCX_F64: return tconv_forward_t<double>(x, map, iw, w, bias, y, d, interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" size_t mcx_tconv_backward_workspace(int64_t, int64_t, int64_t, int64_t, int64_t,
                                               int64_t, int64_t, int64_t, int64_t, int) {
  return 0;
}

extern "C" int mcx_tconv_backward(const void *gy, const void *map, const void *iw, const void *x,
                                  const void *w, void *gx, void *gw, void *gb, void *workspace,
                                  size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co,
                                  int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                                  int64_t P, int interp, int dtype, void *stream) {
  (void)workspace;
  (void)workspace_bytes;
  const ConvDims d{B, Ci, Co, IH, IW, OH, OW, K, P};
  if (int rc = check_dims(d)) return rc;
  if (int rc = check_ptrs(gy, map, iw, w, P)) return rc;
  if (gw && !x) return MCX_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MCX_F32: return tconv_backward_t<float>(gy, map, iw, x, w, gx, gw, gb, d, interp, s);
    case MCX_F64: return tconv_backward_t<double>(gy, map, iw, x, w, gx, gw, gb, d, interp, s);
    default: return MCX_E_DTYPE;
  }
}

extern "C" int mcx_abi_version(void) { return 1; }

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
