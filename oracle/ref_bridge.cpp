/*
 * ref_bridge.cpp -- C entry points onto the REAL MatConvNet CPU objects.  TEST INFRASTRUCTURE ONLY.
 *
 * This file contains no reference code.  It is compiled together with the reference's own sources
 * where they lie (bits/data.cpp, bits/nnpooling.cpp, bits/nnbnorm.cpp, bits/impl/im2row_cpu.cpp; see
 * the Makefile beside this file) and only wraps raw pointers in vl::Tensor views before calling
 * vl::nn::Pooling, vl::nn::BatchNorm and vl::impl::im2row.  The result, oracle/_ref/libmcnref.so, is
 * what the restated oracle is pinned against.
 *
 * vl::nn::Convolution is NOT bridged: bits/nnconv.cu includes MATLAB's <blas.h> through
 * bits/impl/blashelper.hpp:18 and links libmwblas; neither exists outside a MATLAB installation.
 */
#include "nnbnorm.hpp"
#include "nnpooling.hpp"
#include "impl/im2row.hpp"

#include <stddef.h>

namespace {
template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static const vl::DataType value = vl::VLDT_Float; };
template <> struct dtype_of<double> { static const vl::DataType value = vl::VLDT_Double; };

template <typename T>
vl::Tensor view(const T* p, size_t h, size_t w, size_t c, size_t n) {
  if (!p) return vl::Tensor();
  return vl::Tensor(vl::TensorShape(h, w, c, n), dtype_of<T>::value, vl::VLDT_CPU, (void*)p,
                    sizeof(T) * h * w * c * n);
}

template <typename T>
int pool(int backward, T* out, const T* x, const T* dy, int H, int W, int C, int N, int poolH,
         int poolW, int sy, int sx, int pt, int pb, int pl, int pr, int method) {
  vl::Context ctx;
  vl::nn::Pooling op(ctx, poolH, poolW, sy, sx, pt, pb, pl, pr,
                     method == 0 ? vl::nn::Pooling::Max : vl::nn::Pooling::Average);
  const int outH = (H + pt + pb - poolH) / sy + 1;
  const int outW = (W + pl + pr - poolW) / sx + 1;
  vl::Tensor X = view(x, H, W, C, N);
  if (!backward) {
    vl::Tensor Y = view(out, outH, outW, C, N);
    return (int)op.forward(Y, X);
  }
  vl::Tensor DX = view(out, H, W, C, N);
  vl::Tensor DY = view(dy, outH, outW, C, N);
  return (int)op.backward(DX, X, DY);
}

template <typename T>
int bnorm_fwd(T* y, T* moments, const T* x, const T* g, const T* b, int H, int W, int C, int N,
              double eps, int given) {
  vl::Context ctx;
  vl::nn::BatchNorm op(ctx, eps);
  vl::Tensor Y = view(y, H, W, C, N), X = view(x, H, W, C, N);
  vl::Tensor G = view(g, C, 1, 1, 1), B = view(b, C, 1, 1, 1), M = view(moments, C, 2, 1, 1);
  return (int)(given ? op.forwardWithMoment(Y, M, X, G, B) : op.forward(Y, M, X, G, B));
}

template <typename T>
int bnorm_bwd(T* dx, T* dg, T* db, T* moments, const T* x, const T* g, const T* b, const T* dy,
              int H, int W, int C, int N, double eps, int given) {
  vl::Context ctx;
  vl::nn::BatchNorm op(ctx, eps);
  vl::Tensor DX = view(dx, H, W, C, N), X = view(x, H, W, C, N), DY = view(dy, H, W, C, N);
  vl::Tensor DG = view(dg, C, 1, 1, 1), DB = view(db, C, 1, 1, 1);
  vl::Tensor G = view(g, C, 1, 1, 1), B = view(b, C, 1, 1, 1), M = view(moments, C, 2, 1, 1);
  return (int)(given ? op.backwardWithMoment(DX, DG, DB, M, X, G, B, DY)
                     : op.backward(DX, DG, DB, M, X, G, B, DY));
}
}  // namespace

extern "C" {

#define REF_DEFINE(T, S)                                                                            \
  int ref_pool_forward_##S(T* y, const T* x, int H, int W, int C, int N, int poolH, int poolW,      \
                           int sy, int sx, int pt, int pb, int pl, int pr, int method) {            \
    return pool<T>(0, y, x, (const T*)0, H, W, C, N, poolH, poolW, sy, sx, pt, pb, pl, pr, method); \
  }                                                                                                 \
  int ref_pool_backward_##S(T* dx, const T* x, const T* dy, int H, int W, int C, int N, int poolH,  \
                            int poolW, int sy, int sx, int pt, int pb, int pl, int pr,              \
                            int method) {                                                           \
    return pool<T>(1, dx, x, dy, H, W, C, N, poolH, poolW, sy, sx, pt, pb, pl, pr, method);         \
  }                                                                                                 \
  int ref_bnorm_forward_##S(T* y, T* moments, const T* x, const T* g, const T* b, int H, int W,     \
                            int C, int N, double eps, int given) {                                  \
    return bnorm_fwd<T>(y, moments, x, g, b, H, W, C, N, eps, given);                               \
  }                                                                                                 \
  int ref_bnorm_backward_##S(T* dx, T* dg, T* db, T* moments, const T* x, const T* g, const T* b,   \
                             const T* dy, int H, int W, int C, int N, double eps, int given) {      \
    return bnorm_bwd<T>(dx, dg, db, moments, x, g, b, dy, H, W, C, N, eps, given);                  \
  }                                                                                                 \
  int ref_im2row_forward_##S(T* stacked, const T* data, int H, int W, int C, int FH, int FW,        \
                             int sy, int sx, int pt, int pb, int pl, int pr, int dy, int dx) {      \
    vl::Context ctx;                                                                                \
    return (int)vl::impl::im2row<vl::VLDT_CPU, T>::forward(ctx, stacked, data, H, W, C, FH, FW, sy, \
                                                           sx, pt, pb, pl, pr, dy, dx);             \
  }                                                                                                 \
  int ref_im2row_backward_##S(T* data, const T* stacked, int H, int W, int C, int FH, int FW,       \
                              int sy, int sx, int pt, int pb, int pl, int pr, int dy, int dx) {     \
    vl::Context ctx;                                                                                \
    return (int)vl::impl::im2row<vl::VLDT_CPU, T>::backward(ctx, data, stacked, H, W, C, FH, FW,    \
                                                            sy, sx, pt, pb, pl, pr, dy, dx);        \
  }

REF_DEFINE(float, f32)
REF_DEFINE(double, f64)

}  // extern "C"
