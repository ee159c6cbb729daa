/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain-C CPU restatement of the reference's mapped-convolution hot path
 * (gather / scatter interpolators, mapped im2col + GEMM convolution and its
 * transposed form, mapped max / average pooling, resample / unresample, KNN),
 * instantiated for float (_f32) and double (_f64).  Only tests, the smoke
 * check and the bench's CPU-baseline leg may load the library built from this
 * file; the shipped HIP library never links, loads or falls back to it.
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   - interpolators, resample, conv, transposed conv, pools: the reference's
 *     own hand-computed known answers (literals of the files under package/tests, transcribed
 *     as data), the reference's CPU build in oracle/_ref where present, and
 *     closed forms (torch grid_sample / conv2d special cases, adjointness).
 *   - orc_knn: the reference holds no test, no CPU twin and no runnable wiring
 *     for it -> "parity unpinned" by the reference; pinned by brute force
 *     (stable argsort of the same fused-multiply-add distances) only.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -ffp-contract=off)
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define T float
#define FN(name) CAT(name, _f32)
#define FMA fmaf
#define SQRT sqrtf
#include "mcx_oracle_impl.inc"
#undef T
#undef FN
#undef FMA
#undef SQRT

#define T double
#define FN(name) CAT(name, _f64)
#define FMA fma
#define SQRT sqrt
#include "mcx_oracle_impl.inc"
#undef T
#undef FN
#undef FMA
#undef SQRT

int orc_abi_version(void) { return 1; }
