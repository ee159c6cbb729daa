/*
 * mcx.h -- C ABI of the MI355X (gfx950) mapped-convolution backend.
 *
 * One shared library, libmcx_hip.so, exports the functions below.  They are
 * what the reference's Python layers reach through its pybind modules
 * (`_mapped_convolution_ext._*`), re-cut as plain C: device pointers, sizes and
 * an explicit stream; no tensor types.  Citations name the reference interface
 * each entry point replaces (paths relative to package/ext_modules/).
 *
 * Conventions
 *   - All pointers are DEVICE pointers to contiguous row-major buffers, laid
 *     out exactly like the reference's tensors (NCHW data, [H,W,K,(P,)2] maps).
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *     Calls only enqueue work; they never synchronise or allocate.
 *   - `dtype` selects the data scalar: MCX_F32, MCX_F64, or MCX_BF16
 *     (convolution entry points only; accumulation is fp32).  sample_map and
 *     interp_weights have the data's type for F32/F64 and are float for BF16.
 *   - `interp`: 0 nearest (also any other value), 1 bilinear, 2 bispherical
 *     (include/core/resample.h:62-90).
 *   - `P` is the number of interpolation points per tap: 0 means "no
 *     interp_weights" (iw must be NULL, map is [..,K,2]); P >= 1 selects the
 *     weighted form (map [..,K,P,2], iw [..,K,P]).
 *   - Scatter-type outputs (gx, tconv y, resample_to_map out, unpool gin) are
 *     fully overwritten: the library clears them itself before accumulating.
 *   - Return value: 0 on success; a positive hipError_t if a launch failed; a
 *     negative MCX_E_* for rejected arguments.  Nothing aborts the process.
 *   - Thread safety: concurrent calls on different streams are independent as long as
 *     their output and workspace buffers are.  Two pieces of state live in the library: a
 *     per-thread timing request (mcx_profile_dominant_kernel; consumed or dropped by the
 *     next convolution call of that thread) and the per-GPU scratch array of
 *     mcx_conv_forward_static (calls of that one entry point that overlap on one GPU race).
 */
#ifndef MCX_H_
#define MCX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { MCX_F32 = 0, MCX_F64 = 1, MCX_BF16 = 2 };

enum {
  MCX_OK = 0,
  MCX_E_DTYPE = -1,     /* dtype not supported by this entry point */
  MCX_E_SHAPE = -2,     /* a size is negative, zero where it may not be, or too large */
  MCX_E_NULL = -3,      /* a required pointer is NULL (or iw/P disagree) */
  MCX_E_WORKSPACE = -4, /* workspace missing or too small */
  MCX_E_STATIC_LIMIT = -5, /* needs more scratch than mcx_conv_forward_static's fixed buffer */
  MCX_E_PLAN = -6 /* the plan was not built for this op, map, interpolation or size */
};

/* Library identification; bumps when a signature changes. */
int mcx_abi_version(void);
/* Human-readable text for a return code of any function below. */
const char *mcx_error_string(int code);

/* Measurement aid, no counterpart in the reference.  The next convolution entry point this
 * thread calls records the two caller-owned hipEvent_t handles on its stream right before
 * and right after the launch of its dominant kernel (the gather-product or weight-gradient
 * kernel), leaving out weight packing, map building and partial-sum reduction; the request
 * is consumed by that launch.  NULL, NULL cancels a pending request. */
int mcx_profile_dominant_kernel(void *start_event, void *stop_event);

/* ---- Resample / Unresample ------------------------------------------------ */

/* resample_from_map (+ weighted_resample_from_map):
 * include/nn/layers/resample_layer.h:60-61,85 and weighted_resample_layer.h:78-81;
 * kernels include/nn/cuda/resample.cuh:49-61,124-139.
 * dst[b,c,i,j] = sample(src[b,c,:,:], map[i,j]);  src [B,C,SH,SW], map [MH,MW,(P,)2],
 * iw [MH,MW,P] or NULL, dst [B,C,MH,MW]. */
int mcx_resample_from_map(const void *src, const void *map, const void *iw, void *dst,
                          int64_t B, int64_t C, int64_t SH, int64_t SW, int64_t MH, int64_t MW,
                          int64_t P, int interp, int dtype, void *stream);

/* resample_to_map (+ weighted_resample_to_map):
 * include/nn/layers/resample_layer.h:38-40,83 and weighted_resample_layer.h:49-54;
 * kernels include/nn/cuda/resample.cuh:14-26,85-99.
 * out accumulates every input pixel at map[y_in,x_in] (fully written here, the caller need
 * not clear it); in [B,C,IH,IW], map [IH,IW,(P,)2], out [B,C,OH,OW].
 * With a workspace of mcx_resample_to_map_workspace() bytes the map is turned around once and
 * every output is gathered (no float atomics); with workspace == NULL the op scatters with
 * atomics, as the reference does. */
size_t mcx_resample_to_map_workspace(int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t P,
                                     int interp, int dtype);
int mcx_resample_to_map(const void *in, const void *map, const void *iw, void *out,
                        void *workspace, size_t workspace_bytes, int64_t B, int64_t C, int64_t IH,
                        int64_t IW, int64_t OH, int64_t OW, int64_t P, int interp, int dtype,
                        void *stream);

/* ---- Pooling --------------------------------------------------------------- */

/* mapped_max_pool (+ weighted): include/nn/layers/mapped_max_pooling_layer.h:46-49,101,
 * weighted_mapped_max_pooling_layer.h:42-44; kernels include/nn/cuda/mapped_max_pool.cuh:15-31,99-117.
 * in [B,C,IH,IW], map [OH,OW,K,(P,)2] -> out [B,C,OH,OW], idx int64 [B,C,OH,OW]
 * (element offset of the winning tap inside the flattened map; -1 if none). */
int mcx_max_pool(const void *in, const void *map, const void *iw, void *out, int64_t *idx,
                 int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                 int64_t K, int64_t P, int interp, int dtype, void *stream);

/* mapped_max_unpool (+ weighted): mapped_max_pooling_layer.h:69-73,103,
 * weighted_mapped_max_pooling_layer.h:67-70; kernels mapped_max_pool.cuh:56-70,144-159.
 * gout, idx [B,C,OH,OW] -> gin [B,C,IH,IW] (fully written here).  Workspace as for
 * mcx_resample_to_map: mcx_unpool_workspace() bytes select the gather form, NULL the atomics. */
size_t mcx_unpool_workspace(int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                            int interp, int dtype);
int mcx_max_unpool(const void *gout, const int64_t *idx, const void *map, const void *iw,
                   void *gin, void *workspace, size_t workspace_bytes, int64_t B, int64_t C,
                   int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                   int dtype, void *stream);

/* mapped_avg_pool (+ weighted): include/nn/layers/mapped_avg_pooling_layer.h:42-44,91-94,
 * weighted_mapped_avg_pooling_layer.h:48-52; kernels include/nn/cuda/mapped_avg_pool.cuh:15-27,91-106. */
int mcx_avg_pool(const void *in, const void *map, const void *iw, void *out, int64_t B,
                 int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                 int64_t P, int interp, int dtype, void *stream);

/* mapped_avg_unpool (+ weighted): mapped_avg_pooling_layer.h:64-67,
 * weighted_mapped_avg_pooling_layer.h:75-78; kernels mapped_avg_pool.cuh:50-63,131-145.
 * Workspace: mcx_unpool_workspace() bytes, or NULL for the atomic form. */
int mcx_avg_unpool(const void *gout, const void *map, const void *iw, void *gin, void *workspace,
                   size_t workspace_bytes, int64_t B, int64_t C, int64_t IH, int64_t IW, int64_t OH,
                   int64_t OW, int64_t K, int64_t P, int interp, int dtype, void *stream);

/* ---- Mapped convolution ---------------------------------------------------- */

/* mapped_conv_forward (+ weighted_mapped_conv_forward):
 * include/nn/layers/mapped_convolution_layer.h:64-66,141,
 * weighted_mapped_convolution_layer.h:65-68,153; host driver
 * src/nn/cuda/mapped_convolution_layer.cu:16-73.
 * x [B,Ci,IH,IW], map [OH,OW,K,(P,)2], w [Co,Ci,K], bias [Co] -> y [B,Co,OH,OW].
 * The gather, the product with w and the bias are one fused kernel; no column
 * buffer exists. */
int mcx_conv_forward(const void *x, const void *map, const void *iw, const void *w,
                     const void *bias, void *y, void *workspace, size_t workspace_bytes,
                     int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                     int64_t OW, int64_t K, int64_t P, int interp, int dtype, void *stream);

/* mcx_conv_forward for callers that cannot allocate device memory or hand over a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same arguments and results as mcx_conv_forward, but
 * the scratch (repacked weights, the map's pair mask, staging copies) lives in an array of
 * MCX_STATIC_SCRATCH_BYTES inside the library's code object, one copy per GPU, held until the
 * process ends; the call makes no hipMalloc / hipFree.  Problems whose
 * mcx_conv_forward_workspace() exceeds that size (bf16 storage and single-row sources need a
 * staging copy as large as the input) return MCX_E_STATIC_LIMIT.  All calls on one GPU share
 * the array: calls that overlap on one GPU (different streams or threads) race; calls on one
 * stream are ordered and safe.  The first call on a device looks up the array's address
 * (hipGetSymbolAddress), so make it outside any graph capture. */
#define MCX_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
int mcx_conv_forward_static(const void *x, const void *map, const void *iw, const void *w,
                            const void *bias, void *y, int64_t B, int64_t Ci, int64_t Co,
                            int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                            int interp, int dtype, void *stream);

/* Bytes of device scratch the matching call needs for these sizes (may be 0).
 * The scratch holds repacked weights, partial sums, staging copies of operands and
 * resolved taps; its contents need not survive the call.  It must be 256-byte aligned. */
size_t mcx_conv_forward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                                  int64_t OH, int64_t OW, int64_t K, int64_t P, int dtype);
size_t mcx_conv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                                   int64_t OH, int64_t OW, int64_t K, int64_t P, int dtype);

/* mapped_conv_backward (+ weighted): mapped_convolution_layer.h:90-135,143,
 * weighted_mapped_convolution_layer.h:97-100,156; host drivers
 * src/nn/cuda/mapped_convolution_layer.cu:75-193.
 * gy [B,Co,OH,OW], x, w as above -> gx [B,Ci,IH,IW] (cleared here),
 * gw [Co,Ci,K], gb [Co] (= gy summed over b,h,w).  Any of gx, gw, gb may be
 * NULL to skip that gradient.  workspace: device scratch of at least
 * mcx_conv_backward_workspace(...) bytes. */
int mcx_conv_backward(const void *gy, const void *map, const void *iw, const void *x,
                      const void *w, void *gx, void *gw, void *gb, void *workspace,
                      size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                      int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                      int dtype, void *stream);

/* mapped_transposed_conv_forward (+ weighted):
 * include/nn/layers/mapped_transposed_convolution_layer.h:64-69,148,
 * weighted_mapped_transposed_convolution_layer.h:64-67; host driver
 * src/nn/cuda/mapped_transposed_convolution_layer.cu:53-110.
 * x [B,Ci,IH,IW], map [IH,IW,K,(P,)2] pointing into the OUTPUT, w [Ci,Co,K],
 * bias [Co] -> y [B,Co,OH,OW] (initialised to the bias here, then accumulated). */
int mcx_tconv_forward(const void *x, const void *map, const void *iw, const void *w,
                      const void *bias, void *y, void *workspace, size_t workspace_bytes,
                      int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW, int64_t OH,
                      int64_t OW, int64_t K, int64_t P, int interp, int dtype, void *stream);

size_t mcx_tconv_forward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                                   int64_t OH, int64_t OW, int64_t K, int64_t P, int dtype);
size_t mcx_tconv_backward_workspace(int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                                    int64_t OH, int64_t OW, int64_t K, int64_t P, int dtype);

/* mapped_transposed_conv_backward (+ weighted):
 * mapped_transposed_convolution_layer.h:97-100,150,
 * weighted_mapped_transposed_convolution_layer.h:98-100; host drivers
 * src/nn/cuda/mapped_transposed_convolution_layer.cu:112-220.
 * gy [B,Co,OH,OW] -> gx [B,Ci,IH,IW], gw [Ci,Co,K], gb [Co]; NULL skips. */
int mcx_tconv_backward(const void *gy, const void *map, const void *iw, const void *x,
                       const void *w, void *gx, void *gw, void *gb, void *workspace,
                       size_t workspace_bytes, int64_t B, int64_t Ci, int64_t Co, int64_t IH,
                       int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                       int dtype, void *stream);

/* ---- Map plans ---------------------------------------------------------------- */

/* A plan is device memory the caller owns; what it was built for is recorded on the HOST, in a
 * descriptor the *_plan_build call fills and the caller hands back with the plan.  Every
 * *_planned entry point compares the descriptor with its own arguments before it enqueues
 * anything - the operation the plan serves, interpolation (as the library canonicalises it),
 * sizes, K, P, the data type where the plan depends on it, the address and size of the plan
 * and, where the entry point also takes the map, the addresses of sample_map and
 * interp_weights the plan was built from - and returns MCX_E_PLAN on any difference, so a plan
 * of equal size built for another map or another interpolation cannot be used by mistake.  The
 * descriptor is plain data (no pointers are followed); `check` folds the other fields so that an
 * uninitialised or edited descriptor is refused too.  A plan is bound to the buffers it was
 * built at and from: after copying a plan or a map elsewhere, build again.  The library cannot
 * see writes into the map: rebuild the plan when the map's contents change. */
enum {
  MCX_PLAN_CONV = 1,       /* mcx_conv_plan_build */
  MCX_PLAN_SCATTER = 2,    /* mcx_scatter_plan_build, for_max_unpool == 0 */
  MCX_PLAN_SCATTER_MAX = 3 /* mcx_scatter_plan_build, for_max_unpool != 0 */
};
typedef struct mcx_plan_desc {
  uint32_t magic; /* 0x4d435850 */
  int32_t kind;   /* MCX_PLAN_* */
  int32_t interp; /* 0 nearest, 1 bilinear, 2 bispherical */
  int32_t dtype;  /* scatter plans hold weights in the data's type (MCX_F32 / MCX_F64); conv: MCX_F32 */
  int64_t SH, SW; /* the image the map points into */
  int64_t MH, MW; /* the map's spatial size */
  int64_t K, P;
  uint64_t plan; /* device address the plan was built at */
  uint64_t plan_bytes;
  uint64_t map, iw; /* device addresses of sample_map and interp_weights (0: none) */
  uint64_t check;
} mcx_plan_desc;

/* Map plan: no counterpart in the reference, which decodes sample_map inside its kernels at
 * every call.  A network applies the same sample_map at every step, so everything that depends
 * on the map alone can be built once and reused: the transposed map of the scatter direction
 * (convolution backward-input, transposed-convolution forward), the taps of the gather
 * direction resolved to (offset, weight) pairs (convolution forward, transposed-convolution
 * backward-input; maps of at most four pairs per tap), and the "which pairs are in use" masks
 * (all of them and the weight gradients).  A plan belongs to one (sample_map, interp_weights,
 * interp, sampled image, map size, K, P).  In mcx_conv_plan_bytes / _build, IH x IW is the image
 * the map samples and OH x OW the map's spatial size: a convolution passes its input and
 * output sizes, a transposed convolution its OUTPUT size as (IH, IW) and its INPUT size as
 * (OH, OW).  The caller rebuilds the plan when the map's contents change.  mcx_conv_plan_bytes
 * is 0 where no plan exists (F64, P > 4): pass NULL, 0 then.  The _planned entry points are the
 * plain ones with the plan in place of the per-call build (plan NULL: identical to the plain
 * call); they only read the plan, so one plan may serve concurrent calls. */
size_t mcx_conv_plan_bytes(int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                           int dtype);
int mcx_conv_plan_build(const void *map, const void *iw, void *plan, size_t plan_bytes,
                        mcx_plan_desc *desc, int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                        int64_t K, int64_t P, int interp, int dtype, void *stream);
int mcx_conv_forward_planned(const void *x, const void *map, const void *iw, const void *w,
                             const void *bias, void *y, void *workspace, size_t workspace_bytes,
                             const void *plan, size_t plan_bytes, const mcx_plan_desc *desc,
                             int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                             int64_t OH, int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                             void *stream);
int mcx_conv_backward_planned(const void *gy, const void *map, const void *iw, const void *x,
                              const void *w, void *gx, void *gw, void *gb, void *workspace,
                              size_t workspace_bytes, const void *plan, size_t plan_bytes,
                              const mcx_plan_desc *desc, int64_t B, int64_t Ci, int64_t Co,
                              int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P,
                              int interp, int dtype, void *stream);
int mcx_tconv_forward_planned(const void *x, const void *map, const void *iw, const void *w,
                              const void *bias, void *y, void *workspace, size_t workspace_bytes,
                              const void *plan, size_t plan_bytes, const mcx_plan_desc *desc,
                              int64_t B, int64_t Ci, int64_t Co, int64_t IH, int64_t IW,
                              int64_t OH, int64_t OW, int64_t K, int64_t P, int interp, int dtype,
                              void *stream);
int mcx_tconv_backward_planned(const void *gy, const void *map, const void *iw, const void *x,
                               const void *w, void *gx, void *gw, void *gb, void *workspace,
                               size_t workspace_bytes, const void *plan, size_t plan_bytes,
                               const mcx_plan_desc *desc, int64_t B, int64_t Ci, int64_t Co,
                               int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                               int64_t P, int interp, int dtype, void *stream);

/* Scatter plans: no counterpart in the reference.  resample_to_map and the two unpoolings run
 * as gathers through the transposed form of their sample map (per destination pixel the sorted
 * list of (source, weight) contributions); built per call that is a third of a call's time, and
 * it depends on the map alone.  mcx_scatter_plan_build writes it once into a caller-owned buffer
 * of mcx_scatter_plan_bytes(); the _planned entry points take it in place of (map, iw,
 * workspace) and only read it.  MH x MW: the sample map's spatial size (the source of the
 * scatter); DH x DW: the image scattered into; K = 1 for resample_to_map.  A plan built with
 * for_max_unpool != 0 records the tap of every contribution and serves mcx_max_unpool_planned
 * only; one built with 0 serves the other two.  F32 and F64. */
size_t mcx_scatter_plan_bytes(int64_t MH, int64_t MW, int64_t DH, int64_t DW, int64_t K, int64_t P,
                              int interp, int dtype);
int mcx_scatter_plan_build(const void *map, const void *iw, void *plan, size_t plan_bytes,
                           mcx_plan_desc *desc, int64_t MH, int64_t MW, int64_t DH, int64_t DW,
                           int64_t K, int64_t P, int interp, int dtype, int for_max_unpool,
                           void *stream);
int mcx_resample_to_map_planned(const void *in, const void *plan, size_t plan_bytes,
                                const mcx_plan_desc *desc, void *out, int64_t B, int64_t C,
                                int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t P,
                                int interp, int dtype, void *stream);
int mcx_avg_unpool_planned(const void *gout, const void *plan, size_t plan_bytes,
                           const mcx_plan_desc *desc, void *gin, int64_t B, int64_t C, int64_t IH,
                           int64_t IW, int64_t OH, int64_t OW, int64_t K, int64_t P, int interp,
                           int dtype, void *stream);
int mcx_max_unpool_planned(const void *gout, const int64_t *idx, const void *plan,
                           size_t plan_bytes, const mcx_plan_desc *desc, void *gin, int64_t B,
                           int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t K,
                           int64_t P, int interp, int dtype, void *stream);

/* ---- KNN -------------------------------------------------------------------- */

/* knn_forward: include/util/layers/knn_layer.h:25-35,41; kernels
 * include/util/cuda/knn.cuh:43-275; host src/util/cuda/knn_layer.cu:13-32.
 * ref [B,D,R], query [B,D,Q] (points are columns) -> idx int64 [B,k,Q]
 * (1-based reference index, row j = j-th nearest, ties keep the lower index),
 * dist [B,k,Q] (Euclidean).  k <= 64; F32 and F64.  The R x Q distance matrix
 * of the reference is never formed.
 * workspace (optional): mcx_knn_workspace(B, D, R, dtype) bytes, nonzero for points of one to
 * three dimensions and at least 512 reference points.  With it the reference points are
 * binned into a uniform grid and every query only visits the cells around it; the result is
 * the same bit for bit (same distance arithmetic, same order among equal distances).
 * Without it (NULL) every query walks every reference point. */
size_t mcx_knn_workspace(int64_t B, int64_t D, int64_t R, int dtype);
int mcx_knn(const void *ref, const void *query, int64_t *idx, void *dist, void *workspace,
            size_t workspace_bytes, int64_t B, int64_t D, int64_t R, int64_t Q, int64_t k,
            int dtype, void *stream);

/* ---- sample-map builders and cube-map resampling ----------------------------- */

enum {
  MCX_PROJ_GRID = 0,            /* lon/lat grid in radians: grid_projection_map */
  MCX_PROJ_GNOMONIC = 1,        /* reverse_gnomonic_projection_map + convert_spherical_to_image */
  MCX_PROJ_EQUIRECTANGULAR = 2, /* reverse_equirectangular_projection_map + conversion */
  MCX_PROJ_PERSPECTIVE = 3      /* perspective_projection_map (the pixel grid) */
};

/* get_projection_map / get_perspective_projection_map:
 * package/layers/util/spherical_projections.py:12-24, 33-35 (builders :39-193,
 * conversion package/layers/util/conversions.py:6-17).  Writes the float sample map
 * [ceil(H/stride), ceil(W/stride), kh*kw, 2] of an H x W equirectangular (or, for
 * MCX_PROJ_PERSPECTIVE, plain) image, (x, y) last, on the device.  `dilation` is used
 * by GRID and PERSPECTIVE only, like in the reference.  Entries are evaluated in double
 * and rounded once.  H >= 2 for the three spherical projections; at most 65535 output
 * rows. */
int mcx_projection_map(float *out, int64_t H, int64_t W, int64_t kh, int64_t kw, int proj,
                       int64_t stride, int64_t dilation, void *stream);

/* get_reverse_cube_projection_map: spherical_projections.py:26-30 (:261-311,
 * conversions.py:20-181, grids.py:23-37).  Float sample map
 * [ceil(dim/stride), ceil(6*dim/stride), kh*kw, 2] into the dim x 6*dim cube-map image
 * with faces [-z, -x, +z, +x, +y, -y]. */
int mcx_cube_projection_map(float *out, int64_t cube_dim, int64_t kh, int64_t kw, int64_t stride,
                            void *stream);

/* cube2rect: include/util/layers/cube2rect_layer.h:29-43, kernel
 * include/util/cuda/cube2rect.cuh:16-64, host src/util/cuda/cube2rect_layer.cu:11-29.
 * cubemap [C, dim, 6*dim] -> rect [C, RH, RW]; interp 1 bilinear, anything else nearest;
 * F32 and F64. */
int mcx_cube2rect(const void *cubemap, void *rect, int64_t C, int64_t cube_dim, int64_t RH,
                  int64_t RW, int interp, int dtype, void *stream);

/* ---- icosphere map operators -------------------------------------------------- */

/* gnomonic_kernel: package/layers/util/icosphere_functions.py:135-183.  A kh x kw grid of
 * spacing (res_lon, res_lat) on the plane tangent to the unit sphere at each of V points
 * centres [V, 2] = (longitude, latitude) in radians, carried back onto the sphere:
 * out [V, kh*kw, 2] = (longitude in [-pi, pi), latitude).  The tap of index
 * (kh/2)*kw + kw/2 is the centre itself.  Entries are evaluated in double and rounded once. */
int mcx_gnomonic_samples(const float *centres, float *out, int64_t V, int64_t kh, int64_t kw,
                         double res_lat, double res_lon, void *stream);

/* get_planar_conv_operator_from_samples: package/ext_modules/include/util/cpp/sphere.h:131-175
 * (binding), package/ext_modules/src/util/cpp/sphere.cpp:1117-1270 (driver), :1055-1105
 * (Sphere::_isPointInFace), :1007-1053 (face search); Python caller
 * package/layers/util/icosphere_functions.py:226-262.  For each of N sample directions
 * samples [N, 2] = (longitude, latitude) in radians: the face of the triangle mesh
 * (vertices [V, 3] float, faces [F, 3] int64, a closed mesh around the origin) that the ray
 * pierces -> face_idx [N] int64 (-1: none), vertex_idx [N, 3] int64 (the face's vertices in
 * reverse order, as the reference lists them) and weights [N, 3] float (barycentric s, t, u of
 * the pierced point; `nearest` != 0: one-hot at the largest).  The mesh is the caller's: the
 * reference's own module walks its private icosphere hierarchy on the host; to reproduce it
 * pass the vertices and faces of that icosphere.  Where a sample is within the face test's
 * tolerance (1e-3) of an edge, several faces pass; this library returns the one it lies
 * deepest inside.  workspace: mcx_planar_conv_operator_workspace(F) bytes. */
size_t mcx_planar_conv_operator_workspace(int64_t F);
int mcx_planar_conv_operator(const float *samples, const float *vertices, const int64_t *faces,
                             int64_t *face_idx, int64_t *vertex_idx, float *weights,
                             void *workspace, size_t workspace_bytes, int64_t N, int64_t V,
                             int64_t F, int nearest, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MCX_H_ */
