// Element-wise companions of the operators: ReLU, sum of two tensors, scaled sum and the SGD step built from it, fill.  Pure streaming kernels:
// 16-byte accesses, grid-stride, enough workgroups to cover the chip several times.
#include "mcn_internal.hpp"

#include <algorithm>

// Every multiply and add below must stay a separate IEEE operation: results are compared bit for bit
// with the reference CPU loops, so fused multiply-add contraction is switched off for this file.
#pragma clang fp contract(off)

namespace mcn {
namespace {

enum { OP_RELU_FWD, OP_RELU_BWD, OP_ADD, OP_FILL, OP_AXPBY, OP_LRELU_FWD, OP_LRELU_BWD };

template <int OP>
struct Reads {
  static constexpr bool a = OP != OP_FILL;
  static constexpr bool b = OP == OP_RELU_BWD || OP == OP_ADD || OP == OP_AXPBY || OP == OP_LRELU_BWD;
};

template <int OP>
__device__ __forceinline__ float apply1(float a, float b, float k, float k2) {
  switch (OP) {
    case OP_AXPBY: {                                     // scal, then axpy: three roundings like the BLAS pair
      const float t = k * a;
      return t + k2 * b;
    }
    case OP_RELU_FWD: return a > 0.f ? a : 0.f;          // max(x, 0)
    case OP_RELU_BWD: return a > 0.f ? b : b * 0.f;      // dzdy .* (x > 0): keeps NaN/inf*0 semantics
    case OP_ADD: return a + b;
    // leaky: x .* (leak + (1 - leak)*(x > 0)); k = single(leak), k2 = single(leak + (1 - leak)), the two values the
    // factor takes (the reference forms it in double and the product in single, matlab/vl_nnrelu.m:49-55)
    case OP_LRELU_FWD: return a * (a > 0.f ? k2 : k);
    case OP_LRELU_BWD: return b * (a > 0.f ? k2 : k);
    default: return k;
  }
}

// y = op(a, b).  The vector body covers n/4 float4s; the tail (n % 4) is handled by the first threads.
template <int OP, bool VEC4>
__global__ __launch_bounds__(256) void eltwise_kernel(float* __restrict__ y, const float* __restrict__ a,
                                                      const float* __restrict__ b, float k, float k2, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (VEC4) {
    const size_t n4 = n / 4;
    for (size_t i = t; i < n4; i += stride) {
      float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u, r;
      if (Reads<OP>::a) u = stream_load4((const float4*)a + i);
      if (Reads<OP>::b) v = stream_load4((const float4*)b + i);
      r.x = apply1<OP>(u.x, v.x, k, k2);
      r.y = apply1<OP>(u.y, v.y, k, k2);
      r.z = apply1<OP>(u.z, v.z, k, k2);
      r.w = apply1<OP>(u.w, v.w, k, k2);
      stream_store4((float4*)y + i, r);
    }
    for (size_t i = n4 * 4 + t; i < n; i += stride) {
      const float u = Reads<OP>::a ? a[i] : 0.f;
      const float v = Reads<OP>::b ? b[i] : 0.f;
      y[i] = apply1<OP>(u, v, k, k2);
    }
  } else {
    for (size_t i = t; i < n; i += stride) {
      const float u = Reads<OP>::a ? a[i] : 0.f;
      const float v = Reads<OP>::b ? b[i] : 0.f;
      y[i] = apply1<OP>(u, v, k, k2);
    }
  }
}

// SGD with momentum over an arena of parameters: one workgroup per chunk of 1024 elements, every chunk inside one
// parameter, whose rates come from a table.  Each element goes through the roundings of the three scaled sums the
// reference performs one parameter at a time.
__global__ __launch_bounds__(256) void sgd_momentum_kernel(float* __restrict__ value, float* __restrict__ state,
                                                           const float* __restrict__ der,
                                                           const unsigned short* __restrict__ chunkParam,
                                                           const double* __restrict__ rates, double learningRate,
                                                           double weightDecay, float momentum, float derScale, int nesterov) {
  const int p = chunkParam[blockIdx.x];
  const float lr = (float)(learningRate * rates[2 * p]), decay = (float)(weightDecay * rates[2 * p + 1]);
  if (!(lr > 0.f || decay > 0.f)) return;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const float4 v = stream_load4((const float4*)value + i), g = stream_load4((const float4*)der + i);
  const float4 m = stream_load4((const float4*)state + i);
  float4 vo, mo;
  auto one = [&](float v1, float g1, float m1, float& vOut, float& mOut) {
    const float t = derScale * g1;
    const float d = t + decay * v1;      // gradient, normalised, plus weight decay
    const float u = momentum * m1;
    const float mNew = u + (-1.f) * d;   // momentum
    float delta = mNew;
    if (nesterov) delta = momentum * mNew - d;
    const float w = 1.f * v1;
    vOut = w + lr * delta;
    mOut = mNew;
  };
  one(v.x, g.x, m.x, vo.x, mo.x);
  one(v.y, g.y, m.y, vo.y, mo.y);
  one(v.z, g.z, m.z, vo.z, mo.z);
  one(v.w, g.w, m.w, vo.w, mo.w);
  stream_store4((float4*)state + i, mo);
  stream_store4((float4*)value + i, vo);
}

template <int OP>
int launch(const char* who, mcn_stream_t stream, float* y, const float* a, const float* b, float k, size_t n,
           float k2 = 0.f) {
  if (n == 0) return MCN_SUCCESS;
  if (!y || (Reads<OP>::a && !a) || (Reads<OP>::b && !b)) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  const bool vec = aligned16(y) && (!Reads<OP>::a || aligned16(a)) && (!Reads<OP>::b || aligned16(b));
  // each thread handles a few float4s; cap the grid at 32 workgroups per CU-equivalent (256 CUs)
  const size_t work = vec ? (n + 3) / 4 : n;
  const unsigned blocks = (unsigned)std::min<size_t>((work + 255) / 256, 256u * 32u);
  KernelTimer timer("eltwise_kernel", as_stream(stream));
  if (vec) hipLaunchKernelGGL((eltwise_kernel<OP, true>), dim3(blocks), dim3(256), 0, as_stream(stream), y, a, b, k, k2, n);
  else hipLaunchKernelGGL((eltwise_kernel<OP, false>), dim3(blocks), dim3(256), 0, as_stream(stream), y, a, b, k, k2, n);
  return check_launch(who);
}

// y = alpha*a + beta*b in double, each element with the roundings of the reference's scal + axpy pair:
// t = fl(alpha*a), y = fl(t + fl(beta*b))  (this file is compiled without contraction)
__global__ __launch_bounds__(256) void taccum64_kernel(double* __restrict__ y, double alpha, const double* __restrict__ a,
                                                       double beta, const double* __restrict__ b, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const double t = alpha * a[i];
    const double u = beta * b[i];
    y[i] = t + u;
  }
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

int mcn_relu_forward(mcn_stream_t stream, float* y, const float* x, size_t n) {
  return launch<OP_RELU_FWD>("mcn_relu_forward", stream, y, x, nullptr, 0.f, n);
}
int mcn_relu_forward_leaky(mcn_stream_t stream, float* y, const float* x, size_t n, double leak) {
  if (leak == 0) return launch<OP_RELU_FWD>("mcn_relu_forward_leaky", stream, y, x, nullptr, 0.f, n);
  return launch<OP_LRELU_FWD>("mcn_relu_forward_leaky", stream, y, x, nullptr, (float)leak, n, (float)(leak + (1.0 - leak)));
}
int mcn_relu_backward_leaky(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, size_t n,
                            double leak) {
  if (leak == 0) return launch<OP_RELU_BWD>("mcn_relu_backward_leaky", stream, derInput, x, derOutput, 0.f, n);
  return launch<OP_LRELU_BWD>("mcn_relu_backward_leaky", stream, derInput, x, derOutput, (float)leak, n,
                              (float)(leak + (1.0 - leak)));
}
int mcn_relu_backward(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, size_t n) {
  return launch<OP_RELU_BWD>("mcn_relu_backward", stream, derInput, x, derOutput, 0.f, n);
}
int mcn_add(mcn_stream_t stream, float* y, const float* a, const float* b, size_t n) {
  return launch<OP_ADD>("mcn_add", stream, y, a, b, 0.f, n);
}
int mcn_taccum(mcn_stream_t stream, float* y, float alpha, const float* a, float beta, const float* b, size_t n) {
  return launch<OP_AXPBY>("mcn_taccum", stream, y, a, b, alpha, n, beta);
}
int mcn_taccum_f64(mcn_stream_t stream, double* y, double alpha, const double* a, double beta, const double* b, size_t n) {
  if (n == 0) return MCN_SUCCESS;
  if (!y || !a || !b) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_taccum_f64: null tensor");
  const size_t blocks = std::min<size_t>((n + 255) / 256, 256u * 32u);
  KernelTimer timer("taccum64_kernel", as_stream(stream));
  hipLaunchKernelGGL(taccum64_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), y, alpha, a, beta, b, n);
  return check_launch("mcn_taccum_f64");
}
int mcn_sgd_momentum(mcn_stream_t stream, float* value, float* state, const float* der, size_t chunks,
                     const unsigned short* chunkParam, const double* rates, double learningRate, double weightDecay,
                     double momentum, double derScale, int nesterov) {
  if (chunks == 0) return MCN_SUCCESS;
  if (!value || !state || !der || !chunkParam || !rates) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_sgd_momentum: null argument");
  if (!aligned16(value) || !aligned16(state) || !aligned16(der))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_sgd_momentum: the arenas must be 16-byte aligned");
  if (chunks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "mcn_sgd_momentum: arena too large");
  KernelTimer timer("sgd_momentum_kernel", as_stream(stream));
  hipLaunchKernelGGL(sgd_momentum_kernel, dim3((unsigned)chunks), dim3(256), 0, as_stream(stream), value, state, der,
                     chunkParam, rates, learningRate, weightDecay, (float)momentum, (float)derScale, nesterov ? 1 : 0);
  return check_launch("mcn_sgd_momentum");
}
int mcn_fill(mcn_stream_t stream, float* y, float value, size_t n) {
  return launch<OP_FILL>("mcn_fill", stream, y, nullptr, nullptr, value, n);
}

}  // extern "C"
