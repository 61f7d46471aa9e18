/*
 * oracle.h -- CPU restatement of MatConvNet's backward-pass hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library may call, link or
 * load this code: it exists so that tests and the CPU-baseline leg of the
 * benchmark have an independent statement of what the reference computes.
 *
 * All tensors are MATLAB column-major H x W x C x N: element (h,w,c,n) lives at
 * h + H*(w + W*(c + C*n)).  Filters are FH x FW x FC x K in the same order.
 *
 * Each function names the reference source (path:line under the MatConvNet
 * tree, matlab/src/) whose arithmetic and summation order it follows.
 *
 * Pinning status (what independent evidence fixes each function):
 *   pool_forward / pool_backward   -- bit-compared with the compiled reference
 *                                     objects (oracle/_ref) incl. ties, NaN, -inf,
 *                                     clipped windows; torch max/avg_pool2d autograd.
 *   bnorm_*                        -- bit-compared with oracle/_ref (float and
 *                                     double); closed forms of doc/blocks.tex; torch
 *                                     batch_norm autograd in double.
 *   im2row_forward / im2row_backward -- bit-compared with oracle/_ref
 *                                     (impl/im2row_cpu.cpp compiles stand-alone).
 *   conv_forward / conv_backward   -- the reference's conv driver needs MATLAB's
 *                                     <blas.h>/libmwblas (Intel MKL, version tied to the
 *                                     MATLAB release), which is absent, so the real
 *                                     object cannot be built.  Pinned instead by: the
 *                                     real im2row (above), sgemm against numpy matmul,
 *                                     a direct 7-loop convolution gradient in double,
 *                                     torch conv2d autograd in double, adjoint identities,
 *                                     and the stride/pad/group equivalences of
 *                                     matlab/xtest/suite/nnconv.m:88-161.  Only the
 *                                     summation order inside a GEMM is unpinned (it lives
 *                                     in MKL); the parity gate for conv is 2e-4 relative.
 *   subsample_*                    -- bits/nnsubsample.cu needs the same <blas.h> (bias via
 *                                     GEMM with a ones vector), so it cannot be built either.
 *                                     Pinned by the reference's own definition -- empty
 *                                     FILTERS "pretend the identity filter bank"
 *                                     (vl_nnconv.cu:316-321): equal to oracle conv with
 *                                     identity 1x1 filters, forward and backward, bit for bit
 *                                     (tests/test_oracle_conv.py), plus brute force.
 *   convolution transpose          -- composed in oracle/binding.py from conv_backward /
 *                                     conv_forward exactly as bits/nnconv.cu:323-421 does;
 *                                     pinned against torch conv_transpose2d autograd in
 *                                     double (upsample, crop, groups).
 */
#ifndef MCN_ORACLE_H
#define MCN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Geometry of a convolution call (vl::nn::Convolution members, bits/nnconv.hpp:43-51,
 * plus the tensor sizes the MEX driver validates, vl_nnconv.cu:269-342). */
typedef struct oracle_conv_geom {
  int H, W, C, N;        /* input  x : H x W x C x N                     */
  int FH, FW, FC, K;     /* filters  : FH x FW x FC x K (groups = C/FC)  */
  int strideY, strideX;
  int padTop, padBottom, padLeft, padRight;
  int dilateY, dilateX;
} oracle_conv_geom;

/* Geometry of a pooling call (vl::nn::Pooling members, bits/nnpooling.hpp:39-48). */
typedef struct oracle_pool_geom {
  int H, W, C, N;
  int poolH, poolW;
  int strideY, strideX;
  int padTop, padBottom, padLeft, padRight;
  int method;            /* 0 = max, 1 = average (Pooling::Method) */
} oracle_pool_geom;

int oracle_conv_out_h(const oracle_conv_geom* g);
int oracle_conv_out_w(const oracle_conv_geom* g);
int oracle_pool_out_h(const oracle_pool_geom* g);
int oracle_pool_out_w(const oracle_pool_geom* g);

/* Number of OpenMP threads the built-in sgemm will use. */
int oracle_num_threads(void);

/* Optional external Fortran-style gemm with 64-bit integer arguments
 * (ILP64 OpenBLAS `scipy_sgemm_64_` / `scipy_dgemm_64_`).  NULL restores the built-in. */
void oracle_set_sgemm(void* fn);
void oracle_set_dgemm(void* fn);

#define ORACLE_DECLARE(T, S)                                                              \
  /* column-major C = alpha*op(A)*op(B) + beta*C; the role MKL plays behind               \
     bits/impl/blashelper.hpp:79-116 */                                                    \
  void oracle_gemm_##S(char ta, char tb, int64_t m, int64_t n, int64_t k, T alpha,        \
                       const T* a, int64_t lda, const T* b, int64_t ldb, T beta, T* c,    \
                       int64_t ldc);                                                       \
  /* bits/impl/im2row_cpu.cpp:52-163 and :169-230 (one image) */                          \
  void oracle_im2row_forward_##S(T* stacked, const T* data, const oracle_conv_geom* g);   \
  void oracle_im2row_backward_##S(T* data, const T* stacked, const oracle_conv_geom* g);  \
  /* bits/nnconv.cu:71-157; b may be NULL */                                              \
  void oracle_conv_forward_##S(T* y, T outMult, const T* x, T inMult, const T* f,         \
                               const T* b, const oracle_conv_geom* g);                    \
  /* bits/nnconv.cu:163-317; any of dx, df, db may be NULL (skipped) */                   \
  void oracle_conv_backward_##S(T* dx, T* df, T* db, const T* x, const T* f, const T* dy, \
                                const oracle_conv_geom* g);                               \
  /* bits/nnbnorm.cu:46-71,170-256; moments is C x 2 (means then sigmas) */               \
  void oracle_bnorm_forward_##S(T* y, T* moments, const T* x, const T* mult,              \
                                const T* bias, int H, int W, int C, int N, T epsilon,     \
                                int given_moments);                                        \
  /* bits/nnbnorm.cu:74-164,263-365 */                                                     \
  void oracle_bnorm_backward_##S(T* dx, T* dmult, T* dbias, T* moments, const T* x,       \
                                 const T* mult, const T* dy, int H, int W, int C, int N,  \
                                 T epsilon, int given_moments);                            \
  /* bits/nnpooling.cu:102-142 */                                                          \
  void oracle_pool_forward_##S(T* y, const T* x, const oracle_pool_geom* g);              \
  /* bits/nnpooling.cu:170-214; accumulates into dx like the reference (callers zero it, \
     vl_nnpool.cu:255-259) */                                                              \
  void oracle_pool_backward_##S(T* dx, const T* x, const T* dy, const oracle_pool_geom* g); \
  /* matlab/vl_nnrelu.m:43-48 (leak = 0) */                                                \
  void oracle_relu_forward_##S(T* y, const T* x, size_t n);                               \
  void oracle_relu_backward_##S(T* dx, const T* x, const T* dy, size_t n);                \
  /* matlab/+dagnn/Sum.m:11-17 for two inputs */                                           \
  void oracle_sum_##S(T* y, const T* a, const T* b, size_t n);                            \
  /* bits/nnsubsample.cu:36-117 (vl_nnconv with empty FILTERS); bias may be NULL */        \
  void oracle_subsample_forward_##S(T* y, const T* x, const T* bias, int H, int W, int C, \
                                    int N, int strideY, int strideX, int padTop,           \
                                    int padBottom, int padLeft, int padRight);             \
  /* bits/nnsubsample.cu:125-165 */                                                        \
  void oracle_subsample_backward_##S(T* dx, const T* dy, int H, int W, int C, int N,      \
                                     int strideY, int strideX, int padTop, int padBottom, \
                                     int padLeft, int padRight);                                \
  /* matlab/src/vl_taccummex.cu:48-78: y = a (copy), BLAS scal y *= alpha, BLAS axpy       \
     y += beta*b, as the reference-BLAS loops; y may be a */                               \
  void oracle_taccum_##S(T* y, T alpha, const T* a, T beta, const T* b, size_t n);

ORACLE_DECLARE(float, f32)
ORACLE_DECLARE(double, f64)

#ifdef __cplusplus
}
#endif
#endif
