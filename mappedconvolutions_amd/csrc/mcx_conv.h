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

// ---- matrix-core kernels (mcx_conv_mfma.hip), templated on the storage type TD
// (float or bf16_t; arithmetic and accumulation are fp32 in both cases) -----------
struct bf16_t;
bool mfma_supported(int64_t P);
size_t mfma_gather_product_bytes(int64_t O, int64_t G, int64_t K, int64_t B, int64_t SH,
                                 int64_t SW, int elem, int64_t MH, int64_t MW);
template <typename TD>
int mfma_gather_product(const TD *src, const float *map, const float *iw, const TD *w,
                        const TD *bias, TD *y, void *scratch, int64_t B, int64_t G, int64_t O,
                        int64_t SH, int64_t SW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                        int interp, hipStream_t s, const void *plan = nullptr);
size_t mfma_weight_grad_bytes(int64_t B, int64_t A, int64_t G, int64_t MH, int64_t MW, int64_t K,
                              int64_t GH, int64_t GW, size_t elem);
template <typename TD>
int mfma_weight_grad(const TD *plain, const TD *gath, const float *map, const float *iw, TD *gw,
                     void *scratch, int64_t B, int64_t A, int64_t G, int64_t GH, int64_t GW,
                     int64_t MH, int64_t MW, int64_t K, int64_t P, int interp, hipStream_t s,
                     TD *plain_sum, const void *plan = nullptr);
size_t mfma_product_scatter_bytes(int64_t B, int64_t S, int64_t D, int64_t K, int64_t DH,
                                  int64_t DW, size_t elem, int64_t MH, int64_t MW, int64_t P);
template <typename TD>
int mfma_product_scatter(const TD *src, const float *map, const float *iw, const TD *w,
                         const TD *bias, TD *dst, void *scratch, int64_t B, int64_t S, int64_t D,
                         int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                         int interp, hipStream_t s, const void *plan = nullptr);
// A plan is the transposed map of one sample map (DH x DW: the image the map samples; MH x MW:
// the map), built once and passed to mfma_product_scatter / mfma_weight_grad in place of the
// per-call build.  0 bytes: this shape has no transposed-map path.
size_t mfma_scatter_plan_bytes(int64_t DH, int64_t DW, int64_t MH, int64_t MW, int64_t K,
                               int64_t P);
int mfma_scatter_plan_build(const float *map, const float *iw, void *plan, int64_t DH, int64_t DW,
                            int64_t MH, int64_t MW, int64_t K, int64_t P, int interp,
                            hipStream_t s);
size_t mfma_bias_grad_bytes(int64_t B, int64_t C, int64_t N);
template <typename TD>
int mfma_bias_grad(const TD *g, TD *gb, void *scratch, int64_t B, int64_t C, int64_t N,
                   hipStream_t s);

// One-shot timing of the next gather-product / weight-gradient kernel launched by this thread.
void set_profile_events(void *start, void *stop);

}  // namespace mcx
