/*
 * oracle_ops.cpp -- CPU restatement of MatConvNet's convolution, batch-normalisation and
 * pooling operators (forward and backward).  TEST INFRASTRUCTURE ONLY: see oracle.h.
 *
 * Compiled without FMA contraction and without reassociation so that float results follow the
 * reference's sequential C++ loops operation by operation.
 */
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

namespace {

inline int out_extent(int in, int padA, int padB, int window, int dilate, int stride) {
  /* impl/im2row_cpu.cpp:68-73, vl_nnconv.cu:321-331 */
  const int extent = (window - 1) * dilate + 1;
  return (in + padA + padB - extent) / stride + 1;
}

inline int ceil_div(int a, int b) { return (a >= 0) ? (a + b - 1) / b : -((-a) / b); }
inline int floor_div(int a, int b) { return (a >= 0) ? a / b : -((-a + b - 1) / b); }

template <typename T>
struct gemm_of;
template <>
struct gemm_of<float> {
  static void run(char ta, char tb, int64_t m, int64_t n, int64_t k, float alpha, const float* a,
                  int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc) {
    oracle_gemm_f32(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
  }
};
template <>
struct gemm_of<double> {
  static void run(char ta, char tb, int64_t m, int64_t n, int64_t k, double alpha, const double* a,
                  int64_t lda, const double* b, int64_t ldb, double beta, double* c, int64_t ldc) {
    oracle_gemm_f64(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
  }
};

/* Range of patch indices o in [0,numPatches) whose tap lands inside the image:
   0 <= o*stride + tap*dilate - pad <= size-1  (impl/im2row_cpu.cpp:101-132). */
inline void valid_range(int size, int numPatches, int stride, int pad, int tapOffset, int* o0,
                        int* o1) {
  int lo = ceil_div(pad - tapOffset, stride);
  int hi = floor_div(size - 1 + pad - tapOffset, stride) + 1;
  lo = std::max(0, std::min(numPatches, lo));
  hi = std::max(lo, std::min(numPatches, hi));
  *o0 = lo;
  *o1 = hi;
}

/* ---------------------------------------------------------------- im2row / row2im */

/* Patch matrix of ONE image: stacked[r*P + ow*outH + oh], r = i + FH*(j + FW*d), zero outside the
   image (impl/im2row_cpu.cpp:52-163; that file calls the fast axis "width"). */
template <typename T>
void im2row_forward(T* stacked, const T* data, const oracle_conv_geom& g) {
  const int outH = out_extent(g.H, g.padTop, g.padBottom, g.FH, g.dilateY, g.strideY);
  const int outW = out_extent(g.W, g.padLeft, g.padRight, g.FW, g.dilateX, g.strideX);
  const int rows = g.FH * g.FW * g.C;
  for (int r = 0; r < rows; ++r) {
    const int i = r % g.FH, j = (r / g.FH) % g.FW, d = r / (g.FH * g.FW);
    int oh0, oh1, ow0, ow1;
    valid_range(g.H, outH, g.strideY, g.padTop, i * g.dilateY, &oh0, &oh1);
    valid_range(g.W, outW, g.strideX, g.padLeft, j * g.dilateX, &ow0, &ow1);
    T* dst = stacked + (size_t)r * outH * outW;
    const T* plane = data + (size_t)d * g.H * g.W;
    for (int ow = 0; ow < outW; ++ow) {
      T* col = dst + (size_t)ow * outH;
      if (ow < ow0 || ow >= ow1) {
        for (int oh = 0; oh < outH; ++oh) col[oh] = 0;
        continue;
      }
      const int w = ow * g.strideX + j * g.dilateX - g.padLeft;
      const T* src = plane + (size_t)w * g.H + (i * g.dilateY - g.padTop);
      for (int oh = 0; oh < oh0; ++oh) col[oh] = 0;
      for (int oh = oh0; oh < oh1; ++oh) col[oh] = src[oh * g.strideY];
      for (int oh = oh1; oh < outH; ++oh) col[oh] = 0;
    }
  }
}

/* Adjoint of the above: zero the image then add patch-matrix rows back in ascending row order, each
   row in ascending (ow, oh) order (impl/im2row_cpu.cpp:169-230). */
template <typename T>
void im2row_backward(T* data, const T* stacked, const oracle_conv_geom& g) {
  const int outH = out_extent(g.H, g.padTop, g.padBottom, g.FH, g.dilateY, g.strideY);
  const int outW = out_extent(g.W, g.padLeft, g.padRight, g.FW, g.dilateX, g.strideX);
  const int rows = g.FH * g.FW * g.C;
  std::memset(data, 0, sizeof(T) * (size_t)g.H * g.W * g.C);
  for (int r = 0; r < rows; ++r) {
    const int i = r % g.FH, j = (r / g.FH) % g.FW, d = r / (g.FH * g.FW);
    int oh0, oh1, ow0, ow1;
    valid_range(g.H, outH, g.strideY, g.padTop, i * g.dilateY, &oh0, &oh1);
    valid_range(g.W, outW, g.strideX, g.padLeft, j * g.dilateX, &ow0, &ow1);
    const T* src = stacked + (size_t)r * outH * outW;
    T* plane = data + (size_t)d * g.H * g.W;
    for (int ow = ow0; ow < ow1; ++ow) {
      const int w = ow * g.strideX + j * g.dilateX - g.padLeft;
      T* dst = plane + (size_t)w * g.H + (i * g.dilateY - g.padTop);
      const T* col = src + (size_t)ow * outH;
      for (int oh = oh0; oh < oh1; ++oh) dst[oh * g.strideY] += col[oh];
    }
  }
}

/* ---------------------------------------------------------------- convolution */

/* bits/nnconv.cu:71-157: per image, per group  Y = outMult*Y + inMult * phi(x) * F, then the bias as
   a rank-one update with an all-ones vector. */
template <typename T>
void conv_forward(T* y, T outMult, const T* x, T inMult, const T* f, const T* b,
                  const oracle_conv_geom& g) {
  const int outH = out_extent(g.H, g.padTop, g.padBottom, g.FH, g.dilateY, g.strideY);
  const int outW = out_extent(g.W, g.padLeft, g.padRight, g.FW, g.dilateX, g.strideX);
  const int64_t P = (int64_t)outH * outW;
  const int groups = g.C / g.FC;
  const int Kg = g.K / groups;
  const int64_t FV = (int64_t)g.FH * g.FW * g.FC;
  std::vector<T> temp((size_t)(P * FV * groups));
  std::vector<T> ones((size_t)P, T(1));
  for (int n = 0; n < g.N; ++n) {
    const T* xn = x + (size_t)n * g.H * g.W * g.C;
    T* yn = y + (size_t)n * P * g.K;
    im2row_forward(temp.data(), xn, g);
    for (int gr = 0; gr < groups; ++gr) {
      gemm_of<T>::run('n', 'n', P, Kg, FV, inMult, temp.data() + P * FV * gr, P,
                      f + FV * Kg * gr, FV, outMult, yn + P * Kg * gr, P);
    }
    if (b) gemm_of<T>::run('n', 'n', P, g.K, 1, T(1), ones.data(), P, b, 1, T(1), yn, P);
  }
}

/* bits/nnconv.cu:163-317.  Images are visited in ascending order; dzdb and dzdf accumulate across
   images with beta = (image > 0); dzdx of an image = row2im( dY_n * F' ). */
template <typename T>
void conv_backward(T* dx, T* df, T* db, const T* x, const T* f, const T* dy,
                   const oracle_conv_geom& g) {
  const int outH = out_extent(g.H, g.padTop, g.padBottom, g.FH, g.dilateY, g.strideY);
  const int outW = out_extent(g.W, g.padLeft, g.padRight, g.FW, g.dilateX, g.strideX);
  const int64_t P = (int64_t)outH * outW;
  const int groups = g.C / g.FC;
  const int Kg = g.K / groups;
  const int64_t FV = (int64_t)g.FH * g.FW * g.FC;
  std::vector<T> temp;
  if (dx || df) temp.resize((size_t)(P * FV * groups));
  for (int n = 0; n < g.N; ++n) {
    const T* dyn = dy + (size_t)n * P * g.K;
    const T beta = (n > 0) ? T(1) : T(0);
    if (db) {
      /* gemv('t', P, K, 1, dY_n, P, ones, 1, beta, db): db[k] = beta*db[k] + sum_p dY_n[p,k] */
      for (int k = 0; k < g.K; ++k) {
        T s = 0;
        const T* col = dyn + (size_t)k * P;
        for (int64_t p = 0; p < P; ++p) s += col[p];
        db[k] = (n > 0) ? db[k] + s : s;
      }
    }
    if (dx) {
      for (int gr = 0; gr < groups; ++gr) {
        gemm_of<T>::run('n', 't', P, FV, Kg, T(1), dyn + P * Kg * gr, P, f + FV * Kg * gr, FV, T(0),
                        temp.data() + P * FV * gr, P);
      }
      im2row_backward(dx + (size_t)n * g.H * g.W * g.C, temp.data(), g);
    }
    if (df) {
      im2row_forward(temp.data(), x + (size_t)n * g.H * g.W * g.C, g);
      for (int gr = 0; gr < groups; ++gr) {
        gemm_of<T>::run('t', 'n', FV, Kg, P, T(1), temp.data() + P * FV * gr, P, dyn + P * Kg * gr, P,
                        beta, df + FV * Kg * gr, FV);
      }
    }
  }
}

/* ---------------------------------------------------------------- batch normalisation */

/* bits/nnbnorm.cu:46-71: one-pass moments, sums taken in T in channel -> image -> pixel order;
   sigma = sqrt(max(0, E[x^2] - mean^2) + epsilon). */
template <typename T>
void bnorm_moments(T* moments, const T* x, int WH, int C, int N, T epsilon) {
  std::memset(moments, 0, sizeof(T) * 2 * (size_t)C);
  const int mass = WH * N;
  for (int c = 0; c < C; ++c)
    for (int n = 0; n < N; ++n) {
      const T* p = x + (size_t)WH * (c + (size_t)C * n);
      for (int i = 0; i < WH; ++i) {
        const T v = p[i];
        moments[c] += v;
        moments[c + C] += v * v;
      }
    }
  for (int c = 0; c < C; ++c) {
    const T mean = moments[c] / mass;
    const T sigma2 = std::max(T(0), moments[c + C] / mass - mean * mean);
    moments[c] = mean;
    moments[c + C] = std::sqrt(sigma2 + epsilon);
  }
}

/* bits/nnbnorm.cu:170-256 */
template <typename T>
void bnorm_forward(T* y, T* moments, const T* x, const T* mult, const T* bias, int H, int W, int C,
                   int N, T epsilon, int given) {
  const int WH = H * W;
  std::vector<T> own;
  T* mom = moments;
  if (!mom) {
    own.resize(2 * (size_t)C);
    mom = own.data();
  }
  if (!given) bnorm_moments(mom, x, WH, C, N, epsilon);
  for (int c = 0; c < C; ++c) {
    const T mean = mom[c], sigma = mom[c + C], bi = bias[c];
    const T coefficient = mult[c] / sigma;
    for (int n = 0; n < N; ++n) {
      const size_t off = (size_t)WH * (c + (size_t)C * n);
      for (int i = 0; i < WH; ++i) y[off + i] = coefficient * (x[off + i] - mean) + bi;
    }
  }
}

/* bits/nnbnorm.cu:74-164 (helpers) and :263-365 (drivers).  When `given` is zero the four running
   sums are taken in one sweep and the moments are written to `moments` (if non-null). */
template <typename T>
void bnorm_backward(T* dx, T* dmult, T* dbias, T* moments, const T* x, const T* mult, const T* dy,
                    int H, int W, int C, int N, T epsilon, int given) {
  const int WH = H * W;
  std::vector<T> own;
  T* mom = moments;
  if (!mom) {
    own.resize(2 * (size_t)C);
    mom = own.data();
  }
  std::memset(dmult, 0, sizeof(T) * (size_t)C);
  std::memset(dbias, 0, sizeof(T) * (size_t)C);
  if (!given) std::memset(mom, 0, sizeof(T) * 2 * (size_t)C);
  for (int c = 0; c < C; ++c)
    for (int n = 0; n < N; ++n) {
      const size_t off = (size_t)WH * (c + (size_t)C * n);
      for (int i = 0; i < WH; ++i) {
        if (!given) {
          mom[c] += x[off + i];
          mom[c + C] += x[off + i] * x[off + i];
        }
        dmult[c] += dy[off + i] * x[off + i];
        dbias[c] += dy[off + i];
      }
    }
  const T mass = T(WH * N);
  for (int c = 0; c < C; ++c) {
    T mean, sigma;
    if (!given) {
      mean = mom[c] / mass;
      const T sigma2 = std::max(T(0), mom[c + C] / mass - mean * mean);
      sigma = std::sqrt(sigma2 + epsilon);
      mom[c] = mean;
      mom[c + C] = sigma;
    } else {
      mean = mom[c];
      sigma = mom[c + C];
    }
    dmult[c] = (dmult[c] - mean * dbias[c]) / sigma;
  }
  for (int c = 0; c < C; ++c) {
    const T mean = mom[c], sigma = mom[c + C];
    const T muz = dbias[c] / mass;
    const T G1 = mult[c] / sigma;
    const T G2 = G1 * dmult[c] / (mass * sigma);
    for (int n = 0; n < N; ++n) {
      const size_t off = (size_t)WH * (c + (size_t)C * n);
      for (int i = 0; i < WH; ++i) dx[off + i] = G1 * (dy[off + i] - muz) - G2 * (x[off + i] - mean);
    }
  }
}

/* ---------------------------------------------------------------- pooling */

struct window {
  int h1, h2, w1, w2;
};

/* Window of output (oh, ow) clipped to the image (bits/nnpooling.cu:121-126,192-197). */
inline window pool_window(const oracle_pool_geom& g, int oh, int ow) {
  window q;
  q.w1 = ow * g.strideX - g.padLeft;
  q.h1 = oh * g.strideY - g.padTop;
  q.w2 = std::min(q.w1 + g.poolW, g.W);
  q.h2 = std::min(q.h1 + g.poolH, g.H);
  q.w1 = std::max(q.w1, 0);
  q.h1 = std::max(q.h1, 0);
  return q;
}

/* bits/nnpooling.cu:102-142 with the accumulators of :33-96.  Max starts from -inf and uses
   std::max(value, x) (NaN in x never replaces value); average multiplies by 1/clipped-area. */
template <typename T>
void pool_forward(T* y, const T* x, const oracle_pool_geom& g) {
  const int outH = (g.H + g.padTop + g.padBottom - g.poolH) / g.strideY + 1;
  const int outW = (g.W + g.padLeft + g.padRight - g.poolW) / g.strideX + 1;
  for (int z = 0; z < g.C * g.N; ++z) {
    const T* xp = x + (size_t)z * g.H * g.W;
    T* yp = y + (size_t)z * outH * outW;
    for (int ow = 0; ow < outW; ++ow)
      for (int oh = 0; oh < outH; ++oh) {
        const window q = pool_window(g, oh, ow);
        if (g.method == 0) {
          T value = -std::numeric_limits<T>::infinity();
          for (int w = q.w1; w < q.w2; ++w)
            for (int h = q.h1; h < q.h2; ++h) value = std::max(value, xp[w * g.H + h]);
          yp[ow * outH + oh] = value;
        } else {
          T value = 0;
          const T scale = T(1) / T((q.h2 - q.h1) * (q.w2 - q.w1));
          for (int w = q.w1; w < q.w2; ++w)
            for (int h = q.h1; h < q.h2; ++h) value += xp[w * g.H + h];
          yp[ow * outH + oh] = value * scale;
        }
      }
  }
}

/* bits/nnpooling.cu:170-214.  Outputs are visited plane by plane, column (ow) ascending then row
   (oh) ascending.  Max: the winner is the first element, scanning the window column by column,
   that is strictly greater than everything before it (start value -inf); a window with no such
   element routes nothing.  Average: every window element receives dzdy * (1/clipped-area). */
template <typename T>
void pool_backward(T* dx, const T* x, const T* dy, const oracle_pool_geom& g) {
  const int outH = (g.H + g.padTop + g.padBottom - g.poolH) / g.strideY + 1;
  const int outW = (g.W + g.padLeft + g.padRight - g.poolW) / g.strideX + 1;
  for (int z = 0; z < g.C * g.N; ++z) {
    const T* xp = x + (size_t)z * g.H * g.W;
    T* dxp = dx + (size_t)z * g.H * g.W;
    const T* dyp = dy + (size_t)z * outH * outW;
    for (int ow = 0; ow < outW; ++ow)
      for (int oh = 0; oh < outH; ++oh) {
        const window q = pool_window(g, oh, ow);
        const T d = dyp[ow * outH + oh];
        if (g.method == 0) {
          T value = -std::numeric_limits<T>::infinity();
          T* winner = nullptr;
          for (int w = q.w1; w < q.w2; ++w)
            for (int h = q.h1; h < q.h2; ++h) {
              const T v = xp[w * g.H + h];
              if (v > value) {
                value = v;
                winner = dxp + w * g.H + h;
              }
            }
          if (winner) *winner += d;
        } else {
          const T scale = T(1) / T((q.h2 - q.h1) * (q.w2 - q.w1));
          for (int w = q.w1; w < q.w2; ++w)
            for (int h = q.h1; h < q.h2; ++h) dxp[w * g.H + h] += d * scale;
        }
      }
  }
}

}  // namespace

// ---------------------------------------------------------------------------------------------------
// Subsampling with bias: what vl_nnconv computes for empty FILTERS (bits/nnsubsample.cu).
// ---------------------------------------------------------------------------------------------------

// bits/nnsubsample.cu:36-72 (sampling) and :88-117 (bias: output += ones * biases', one add per element)
template <typename T>
static void subsample_forward(T* y, const T* x, const T* bias, int H, int W, int Cc, int N, int sy, int sx, int pt,
                              int pb, int pl, int pr) {
  const int outW = (W + (pl + pr) - 1) / sx + 1, outH = (H + (pt + pb) - 1) / sy + 1;
  for (long z = 0; z < (long)Cc * N; ++z) {
    const T* in = x + z * (long)W * H;
    T* out = y + z * (long)outW * outH;
    for (int ox = 0; ox < outW; ++ox)
      for (int oy = 0; oy < outH; ++oy) {
        const int x1 = ox * sx - pl, y1 = oy * sy - pt;
        T value = 0;
        if (x1 >= 0 && x1 < W && y1 >= 0 && y1 < H) value = in[x1 * H + y1];
        out[ox * outH + oy] = bias ? value + bias[z % Cc] : value;
      }
  }
}

// bits/nnsubsample.cu:125-165: zero-fill, then every sampled position receives its output's derivative
template <typename T>
static void subsample_backward(T* dx, const T* dy, int H, int W, int Cc, int N, int sy, int sx, int pt, int pb, int pl,
                               int pr) {
  const int outW = (W + (pl + pr) - 1) / sx + 1, outH = (H + (pt + pb) - 1) / sy + 1;
  std::memset(dx, 0, sizeof(T) * (size_t)W * H * Cc * N);
  for (long z = 0; z < (long)Cc * N; ++z) {
    T* din = dx + z * (long)W * H;
    const T* dout = dy + z * (long)outW * outH;
    for (int px = 0; px < outW; ++px)
      for (int py = 0; py < outH; ++py) {
        const int x1 = px * sx - pl, y1 = py * sy - pt;
        if (x1 >= 0 && x1 < W && y1 >= 0 && y1 < H) din[x1 * H + y1] = dout[px * outH + py];
      }
  }
}

extern "C" {

int oracle_conv_out_h(const oracle_conv_geom* g) {
  return out_extent(g->H, g->padTop, g->padBottom, g->FH, g->dilateY, g->strideY);
}
int oracle_conv_out_w(const oracle_conv_geom* g) {
  return out_extent(g->W, g->padLeft, g->padRight, g->FW, g->dilateX, g->strideX);
}
int oracle_pool_out_h(const oracle_pool_geom* g) {
  return (g->H + g->padTop + g->padBottom - g->poolH) / g->strideY + 1;
}
int oracle_pool_out_w(const oracle_pool_geom* g) {
  return (g->W + g->padLeft + g->padRight - g->poolW) / g->strideX + 1;
}

#define ORACLE_DEFINE(T, S)                                                                        \
  void oracle_im2row_forward_##S(T* stacked, const T* data, const oracle_conv_geom* g) {           \
    im2row_forward<T>(stacked, data, *g);                                                          \
  }                                                                                                \
  void oracle_im2row_backward_##S(T* data, const T* stacked, const oracle_conv_geom* g) {          \
    im2row_backward<T>(data, stacked, *g);                                                         \
  }                                                                                                \
  void oracle_conv_forward_##S(T* y, T outMult, const T* x, T inMult, const T* f, const T* b,      \
                               const oracle_conv_geom* g) {                                        \
    conv_forward<T>(y, outMult, x, inMult, f, b, *g);                                              \
  }                                                                                                \
  void oracle_conv_backward_##S(T* dx, T* df, T* db, const T* x, const T* f, const T* dy,          \
                                const oracle_conv_geom* g) {                                       \
    conv_backward<T>(dx, df, db, x, f, dy, *g);                                                    \
  }                                                                                                \
  void oracle_bnorm_forward_##S(T* y, T* moments, const T* x, const T* mult, const T* bias, int H, \
                                int W, int C, int N, T epsilon, int given) {                       \
    bnorm_forward<T>(y, moments, x, mult, bias, H, W, C, N, epsilon, given);                       \
  }                                                                                                \
  void oracle_bnorm_backward_##S(T* dx, T* dmult, T* dbias, T* moments, const T* x, const T* mult, \
                                 const T* dy, int H, int W, int C, int N, T epsilon, int given) {  \
    bnorm_backward<T>(dx, dmult, dbias, moments, x, mult, dy, H, W, C, N, epsilon, given);         \
  }                                                                                                \
  void oracle_pool_forward_##S(T* y, const T* x, const oracle_pool_geom* g) {                      \
    pool_forward<T>(y, x, *g);                                                                     \
  }                                                                                                \
  void oracle_pool_backward_##S(T* dx, const T* x, const T* dy, const oracle_pool_geom* g) {       \
    pool_backward<T>(dx, x, dy, *g);                                                               \
  }                                                                                                \
  void oracle_relu_forward_##S(T* y, const T* x, size_t n) {                                       \
    for (size_t i = 0; i < n; ++i) y[i] = (x[i] > T(0)) ? x[i] : T(0); /* MATLAB max(NaN,0) = 0 */                                    \
  }                                                                                                \
  void oracle_relu_backward_##S(T* dx, const T* x, const T* dy, size_t n) {                        \
    for (size_t i = 0; i < n; ++i) dx[i] = dy[i] * T(x[i] > T(0));                                 \
  }                                                                                                \
  void oracle_sum_##S(T* y, const T* a, const T* b, size_t n) {                                    \
    for (size_t i = 0; i < n; ++i) y[i] = a[i] + b[i];                                             \
  }                                                                                                \
  void oracle_subsample_forward_##S(T* y, const T* x, const T* bias, int H, int W, int Cc, int N, \
                                    int sy, int sx, int pt, int pb, int pl, int pr) {              \
    subsample_forward<T>(y, x, bias, H, W, Cc, N, sy, sx, pt, pb, pl, pr);                         \
  }                                                                                                \
  void oracle_subsample_backward_##S(T* dx, const T* dy, int H, int W, int Cc, int N, int sy,     \
                                     int sx, int pt, int pb, int pl, int pr) {                     \
    subsample_backward<T>(dx, dy, H, W, Cc, N, sy, sx, pt, pb, pl, pr);                            \
  }                                                                                                \
  void oracle_taccum_##S(T* y, T alpha, const T* a, T beta, const T* b, size_t n) {                \
    for (size_t i = 0; i < n; ++i) y[i] = a[i];               /* copy  */                          \
    for (size_t i = 0; i < n; ++i) y[i] = alpha * y[i];       /* scal  */                          \
    for (size_t i = 0; i < n; ++i) y[i] = y[i] + beta * b[i]; /* axpy  */                          \
  }

ORACLE_DEFINE(float, f32)
ORACLE_DEFINE(double, f64)

}  // extern "C"
