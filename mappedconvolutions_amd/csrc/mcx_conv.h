// Internal interface between the convolution entry points and the kernel
// translation units.  Three operators cover convolution and transposed
// convolution, forward and backward (roles are described in mcx_conv_generic.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mcx {

int fill_f32(float *p, int64_t n, float v, hipStream_t s);
int fill_f64(double *p, int64_t n, double v, hipStream_t s);

template <typename T>
int generic_gather_product(const T *src, const T *map, const T *iw, const T *w, const T *bias,
                           T *y, int64_t B, int64_t G, int64_t O, int64_t SH, int64_t SW,
                           int64_t N, int64_t K, int64_t P, int interp, hipStream_t s);
template <typename T>
int generic_product_scatter(const T *src, const T *map, const T *iw, const T *w, T *dst,
                            int64_t B, int64_t S, int64_t D, int64_t DH, int64_t DW, int64_t N,
                            int64_t K, int64_t P, int interp, hipStream_t s);
template <typename T>
int generic_weight_grad(const T *plain, const T *gath, const T *map, const T *iw, T *gw,
                        int64_t B, int64_t A, int64_t G, int64_t GH, int64_t GW, int64_t N,
                        int64_t K, int64_t P, int interp, hipStream_t s);
// scratch: channel_sum_scratch_bytes(...) bytes, or NULL for the single-kernel form.
size_t channel_sum_scratch_bytes(int64_t B, int64_t C, int64_t N, size_t elem);
template <typename T>
int channel_sum(const T *g, T *gb, T *scratch, int64_t B, int64_t C, int64_t N, hipStream_t s);
template <typename T>
int fill_bias(T *y, const T *bias, int64_t B, int64_t C, int64_t N, hipStream_t s);

// ---- fp32 matrix-core kernels (mcx_conv_mfma_f32.hip) -------------------------
size_t mfma_f32_packed_weight_bytes(int64_t O, int64_t G, int64_t K);
bool mfma_f32_gather_product_supported(int64_t P);
int mfma_f32_gather_product(const float *src, const float *map, const float *iw, const float *w,
                            const float *bias, float *y, float *wp, int64_t B, int64_t G,
                            int64_t O, int64_t SH, int64_t SW, int64_t OH, int64_t OW, int64_t K,
                            int64_t P, int interp, hipStream_t s);

bool mfma_f32_weight_grad_supported(int64_t P);
size_t mfma_f32_weight_grad_bytes(int64_t B, int64_t A, int64_t G, int64_t MH, int64_t MW,
                                  int64_t K);
int mfma_f32_weight_grad(const float *plain, const float *gath, const float *map, const float *iw,
                         float *gw, float *part, int64_t B, int64_t A, int64_t G, int64_t GH,
                         int64_t GW, int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                         hipStream_t s);

bool mfma_f32_product_scatter_supported(int64_t P);
size_t mfma_f32_product_scatter_bytes(int64_t S, int64_t D, int64_t K, int64_t DH, int64_t DW);
int mfma_f32_product_scatter(const float *src, const float *map, const float *iw, const float *w,
                             const float *bias, float *dst, void *scratch, int64_t B, int64_t S,
                             int64_t D, int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,
                             int64_t P, int interp, hipStream_t s);

}  // namespace mcx
