// Subsampling with bias (vl_nnconv with empty FILTERS: the identity filter bank, matlab/src/vl_nnconv.cu:316-321,
// bits/nnsubsample.cu:31-216) and the per-channel bias add used by ConvolutionTranspose
// (bits/nnconv.cu:369-371 -> bits/nnbias.cu).  Pure data movement plus at most one add per element: HBM-bound.
#include "mcn_internal.hpp"

#include <algorithm>

#pragma clang fp contract(off)

namespace mcn {
namespace {

struct SubP {
  int H, W, outH, outW;
  int sy, sx, pt, pl;
  int C;  // channels (bias index = plane % C)
  FastDiv byOutH, byOutW, byH, byW, bySy, bySx, byC;
};

// y[oh, ow, z] = x[oh*sy - pt, ow*sx - pl, z] (0 outside the image) + bias[z % C]   (nnsubsample.cu:56-69,104-116)
template <typename T>
__global__ __launch_bounds__(256) void subsample_forward_kernel(T* __restrict__ y, const T* __restrict__ x,
                                                                const T* __restrict__ bias, SubP p, unsigned total) {
  for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += gridDim.x * 256u) {
    int t, oh, z, ow;
    p.byOutH.divmod((int)idx, &t, &oh);
    p.byOutW.divmod(t, &z, &ow);
    const int h = oh * p.sy - p.pt, w = ow * p.sx - p.pl;
    T v = 0;
    if ((unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W) v = x[((size_t)z * p.W + w) * p.H + h];
    if (bias) {
      int q, c;
      p.byC.divmod(z, &q, &c);
      v = v + bias[c];
    }
    y[idx] = v;
  }
}

// dzdx[h, w, z] = dzdy[(h+pt)/sy, (w+pl)/sx, z] where both divisions are exact and in range, else 0
// (the gather form of the zero-fill + scatter of nnsubsample.cu:145-160; every input is hit by at most one output)
template <typename T>
__global__ __launch_bounds__(256) void subsample_backward_kernel(T* __restrict__ dx, const T* __restrict__ dy, SubP p,
                                                                 unsigned total) {
  for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += gridDim.x * 256u) {
    int t, h, z, w;
    p.byH.divmod((int)idx, &t, &h);
    p.byW.divmod(t, &z, &w);
    int oh, rh, ow, rw;
    p.bySy.divmod(h + p.pt, &oh, &rh);
    p.bySx.divmod(w + p.pl, &ow, &rw);
    T v = 0;
    if (rh == 0 && rw == 0 && oh < p.outH && ow < p.outW) v = dy[((size_t)z * p.outW + ow) * p.outH + oh];
    dx[idx] = v;
  }
}

// y[q, c, n] += bias[c]; one workgroup per (c, n) plane
template <bool VEC4>
__global__ __launch_bounds__(256) void bias_add_kernel(float* __restrict__ y, const float* __restrict__ bias, int Q, int C) {
  const int plane = blockIdx.x;
  const float b = bias[plane % C];
  float* o = y + (size_t)plane * Q;
  if (VEC4) {
    for (int i = threadIdx.x; i < Q / 4; i += 256) {
      float4 v = ((float4*)o)[i];
      v.x = v.x + b; v.y = v.y + b; v.z = v.z + b; v.w = v.w + b;
      ((float4*)o)[i] = v;
    }
  } else {
    for (int i = threadIdx.x; i < Q; i += 256) o[i] = o[i] + b;
  }
}

// the same for double (one element per access)
__global__ __launch_bounds__(256) void bias_add_kernel_f64(double* __restrict__ y, const double* __restrict__ bias, int Q,
                                                           int C) {
  const int plane = blockIdx.x;
  const double b = bias[plane % C];
  double* o = y + (size_t)plane * Q;
  for (int i = threadIdx.x; i < Q; i += 256) o[i] = o[i] + b;
}

int setup(const char* who, int H, int W, int C, int N, int sy, int sx, int pt, int pb, int pl, int pr, SubP* p,
          size_t* inTotal, size_t* outTotal) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if (sy < 1 || sx < 1) return fail(MCN_ILLEGAL_ARGUMENT, "%s: at least one element of STRIDE is smaller than one", who);
  if (pt < 0 || pb < 0 || pl < 0 || pr < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: an element of PAD is negative", who);
  p->H = H; p->W = W; p->C = C;
  p->sy = sy; p->sx = sx; p->pt = pt; p->pl = pl;
  p->outH = H + pt + pb >= 1 ? (H + pt + pb - 1) / sy + 1 : 0;
  p->outW = W + pl + pr >= 1 ? (W + pl + pr - 1) / sx + 1 : 0;
  *inTotal = (size_t)H * W * C * N;
  *outTotal = (size_t)p->outH * p->outW * C * N;
  if (*inTotal >= (1ull << 31) || *outTotal >= (1ull << 31))
    return fail(MCN_UNSUPPORTED, "%s: tensors of 2^31 elements or more are not supported", who);
  p->byOutH = FastDiv(std::max(p->outH, 1));
  p->byOutW = FastDiv(std::max(p->outW, 1));
  p->byH = FastDiv(std::max(H, 1));
  p->byW = FastDiv(std::max(W, 1));
  p->bySy = FastDiv(sy);
  p->bySx = FastDiv(sx);
  p->byC = FastDiv(std::max(C, 1));
  return MCN_SUCCESS;
}

unsigned grid_for(size_t total) { return (unsigned)std::min<size_t>((total + 255) / 256, 256u * 32u); }

template <typename T>
int subsample_forward(const char* who, mcn_stream_t stream, T* y, const T* x, const T* bias, int H, int W, int C, int N,
                      int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  SubP p;
  size_t inTotal, outTotal;
  int rc = setup(who, H, W, C, N, strideY, strideX, padTop, padBottom, padLeft, padRight, &p, &inTotal, &outTotal);
  if (rc) return rc;
  if (outTotal == 0) return MCN_SUCCESS;
  if (!y || (!x && inTotal > 0)) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  KernelTimer timer("subsample_forward_kernel", as_stream(stream));
  hipLaunchKernelGGL(subsample_forward_kernel<T>, dim3(grid_for(outTotal)), dim3(256), 0, as_stream(stream), y, x, bias, p,
                     (unsigned)outTotal);
  return check_launch(who);
}

template <typename T>
int subsample_backward(const char* who, mcn_stream_t stream, T* derInput, const T* derOutput, int H, int W, int C, int N,
                       int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  SubP p;
  size_t inTotal, outTotal;
  int rc = setup(who, H, W, C, N, strideY, strideX, padTop, padBottom, padLeft, padRight, &p, &inTotal, &outTotal);
  if (rc) return rc;
  if (inTotal == 0) return MCN_SUCCESS;
  if (!derInput || (!derOutput && outTotal > 0)) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  KernelTimer timer("subsample_backward_kernel", as_stream(stream));
  hipLaunchKernelGGL(subsample_backward_kernel<T>, dim3(grid_for(inTotal)), dim3(256), 0, as_stream(stream), derInput,
                     derOutput, p, (unsigned)inTotal);
  return check_launch(who);
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

int mcn_subsample_output_size(int H, int W, int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight,
                              int* outH, int* outW) {
  SubP p;
  size_t a, b;
  int rc = setup("mcn_subsample_output_size", H, W, 1, 1, strideY, strideX, padTop, padBottom, padLeft, padRight, &p, &a, &b);
  if (rc) return rc;
  if (outH) *outH = p.outH;
  if (outW) *outW = p.outW;
  return MCN_SUCCESS;
}

int mcn_subsample_forward(mcn_stream_t stream, float* y, const float* x, const float* bias, int H, int W, int C, int N,
                          int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  return subsample_forward<float>("mcn_subsample_forward", stream, y, x, bias, H, W, C, N, strideY, strideX, padTop,
                                  padBottom, padLeft, padRight);
}

int mcn_subsample_backward(mcn_stream_t stream, float* derInput, const float* derOutput, int H, int W, int C, int N,
                           int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  return subsample_backward<float>("mcn_subsample_backward", stream, derInput, derOutput, H, W, C, N, strideY, strideX,
                                   padTop, padBottom, padLeft, padRight);
}

int mcn_subsample_forward_f64(mcn_stream_t stream, double* y, const double* x, const double* bias, int H, int W, int C,
                              int N, int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  return subsample_forward<double>("mcn_subsample_forward_f64", stream, y, x, bias, H, W, C, N, strideY, strideX, padTop,
                                   padBottom, padLeft, padRight);
}

int mcn_subsample_backward_f64(mcn_stream_t stream, double* derInput, const double* derOutput, int H, int W, int C, int N,
                               int strideY, int strideX, int padTop, int padBottom, int padLeft, int padRight) {
  return subsample_backward<double>("mcn_subsample_backward_f64", stream, derInput, derOutput, H, W, C, N, strideY,
                                    strideX, padTop, padBottom, padLeft, padRight);
}

int mcn_bias_add_f64(mcn_stream_t stream, double* y, const double* bias, int H, int W, int C, int N) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bias_add_f64: negative tensor extent");
  const size_t planes = (size_t)C * N, Q = (size_t)H * W;
  if (planes == 0 || Q == 0) return MCN_SUCCESS;
  if (!y || !bias) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bias_add_f64: null tensor");
  if (planes >= (1ull << 31) || Q >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "mcn_bias_add_f64: tensor too large");
  KernelTimer timer("bias_add_kernel", as_stream(stream));
  hipLaunchKernelGGL(bias_add_kernel_f64, dim3((unsigned)planes), dim3(256), 0, as_stream(stream), y, bias, (int)Q, C);
  return check_launch("mcn_bias_add_f64");
}

int mcn_bias_add(mcn_stream_t stream, float* y, const float* bias, int H, int W, int C, int N) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bias_add: negative tensor extent");
  const size_t planes = (size_t)C * N, Q = (size_t)H * W;
  if (planes == 0 || Q == 0) return MCN_SUCCESS;
  if (!y || !bias) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bias_add: null tensor");
  if (planes >= (1ull << 31) || Q >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "mcn_bias_add: tensor too large");
  KernelTimer timer("bias_add_kernel", as_stream(stream));
  if (Q % 4 == 0 && aligned16(y))
    hipLaunchKernelGGL(bias_add_kernel<true>, dim3((unsigned)planes), dim3(256), 0, as_stream(stream), y, bias, (int)Q, C);
  else
    hipLaunchKernelGGL(bias_add_kernel<false>, dim3((unsigned)planes), dim3(256), 0, as_stream(stream), y, bias, (int)Q, C);
  return check_launch("mcn_bias_add");
}

}  // extern "C"
