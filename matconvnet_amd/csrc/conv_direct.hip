// Direct convolution kernels: one accumulator per output element, any stride / dilation / padding /
// filter groups.  They are the general path for geometries the MFMA implicit-GEMM kernels do not cover
// (filter groups, strided backward-data) and define the semantics those kernels are tested against:
//   y[oh,ow,k,n]  = outMult*y + inMult * sum_{i,j,d} x[oh*sy+i*dy-pt, ow*sx+j*dx-pl, g*FC+d, n] f[i,j,d,k] + b[k]
//   dx[h,w,c,n]   = sum_{k in group(c)} sum_{i,j} dy[(h+pt-i*dy)/sy, (w+pl-j*dx)/sx, k, n] f[i,j,c%FC,k]
//   df[i,j,d,k]   = sum_{n,oh,ow} x[oh*sy+i*dy-pt, ow*sx+j*dx-pl, g*FC+d, n] dy[oh,ow,k,n]
//   db[k]         = sum_{n,oh,ow} dy[oh,ow,k,n]
// (bits/nnconv.cu:71-317 with bits/impl/im2row_cpu.cpp:52-230 folded in.)
#include "conv_common.hpp"

#include <algorithm>

namespace mcn {
namespace {

__global__ __launch_bounds__(256) void conv_fwd_direct(float* __restrict__ y, float outMult,
                                                       const float* __restrict__ x, float inMult,
                                                       const float* __restrict__ f,
                                                       const float* __restrict__ b, ConvP p, size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int P = p.outH * p.outW;
  size_t r = idx;
  const int q = (int)(r % P);
  r /= P;
  const int k = (int)(r % p.K);
  const int n = (int)(r / p.K);
  const int ow = q / p.outH, oh = q - ow * p.outH;
  const int g = k / p.Kg;
  const float* xn = x + (size_t)p.H * p.W * ((size_t)p.C * n + (size_t)g * p.FC);
  const float* fk = f + (size_t)p.FH * p.FW * p.FC * k;
  float acc = 0.f;
  for (int d = 0; d < p.FC; ++d)
    for (int j = 0; j < p.FW; ++j) {
      const int w = ow * p.sx + j * p.dx - p.pl;
      if ((unsigned)w >= (unsigned)p.W) continue;
      for (int i = 0; i < p.FH; ++i) {
        const int h = oh * p.sy + i * p.dy - p.pt;
        if ((unsigned)h >= (unsigned)p.H) continue;
        acc = fmaf(xn[h + p.H * (w + (size_t)p.W * d)], fk[i + p.FH * (j + p.FW * d)], acc);
      }
    }
  float r0 = inMult * acc;
  if (outMult != 0.f) r0 = fmaf(outMult, y[idx], r0);
  if (b) r0 += b[k];
  y[idx] = r0;
}

__global__ __launch_bounds__(256) void conv_bwd_data_direct(float* __restrict__ dx, float dxMult,
                                                            const float* __restrict__ f,
                                                            const float* __restrict__ dy, ConvP p,
                                                            size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int HW = p.H * p.W;
  size_t r = idx;
  const int q = (int)(r % HW);
  r /= HW;
  const int c = (int)(r % p.C);
  const int n = (int)(r / p.C);
  const int w = q / p.H, h = q - w * p.H;
  const int g = c / p.FC, d = c - g * p.FC;
  const int P = p.outH * p.outW;
  float acc = 0.f;
  for (int kk = 0; kk < p.Kg; ++kk) {
    const int k = g * p.Kg + kk;
    const float* dyk = dy + (size_t)P * ((size_t)p.K * n + k);
    const float* fk = f + (size_t)p.FH * p.FW * ((size_t)p.FC * k + d);
    for (int j = 0; j < p.FW; ++j) {
      const int aw = w + p.pl - j * p.dx;
      if (aw < 0 || aw % p.sx) continue;
      const int ow = aw / p.sx;
      if (ow >= p.outW) continue;
      for (int i = 0; i < p.FH; ++i) {
        const int ah = h + p.pt - i * p.dy;
        if (ah < 0 || ah % p.sy) continue;
        const int oh = ah / p.sy;
        if (oh >= p.outH) continue;
        acc = fmaf(dyk[oh + p.outH * ow], fk[i + p.FH * j], acc);
      }
    }
  }
  dx[idx] = dxMult != 0.f ? fmaf(dxMult, dx[idx], acc) : acc;
}

// one workgroup per filter element
__global__ __launch_bounds__(256) void conv_bwd_filter_direct(float* __restrict__ df,
                                                              const float* __restrict__ x,
                                                              const float* __restrict__ dy, ConvP p) {
  __shared__ double lds[4];
  size_t r = blockIdx.x;
  const int i = (int)(r % p.FH);
  r /= p.FH;
  const int j = (int)(r % p.FW);
  r /= p.FW;
  const int d = (int)(r % p.FC);
  const int k = (int)(r / p.FC);
  const int g = k / p.Kg;
  const int c = g * p.FC + d;
  const int P = p.outH * p.outW;
  const long long total = (long long)P * p.N;
  double acc = 0.0;
  for (long long m = threadIdx.x; m < total; m += 256) {
    const int n = (int)(m / P);
    const int q = (int)(m - (long long)n * P);
    const int ow = q / p.outH, oh = q - ow * p.outH;
    const int h = oh * p.sy + i * p.dy - p.pt;
    const int w = ow * p.sx + j * p.dx - p.pl;
    if ((unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W)
      acc += (double)(x[h + p.H * (w + (size_t)p.W * (c + (size_t)p.C * n))] *
                      dy[q + (size_t)P * (k + (size_t)p.K * n)]);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) df[blockIdx.x] = (float)((lds[0] + lds[1]) + (lds[2] + lds[3]));
}

}  // namespace

int conv_forward_direct(hipStream_t s, const ConvP& p, float* y, float outMult, const float* x, float inMult,
                        const float* f, const float* b) {
  const size_t total = (size_t)p.outH * p.outW * p.K * p.N;
  const size_t blocks = (total + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "conv forward: tensor too large");
  hipLaunchKernelGGL(conv_fwd_direct, dim3((unsigned)blocks), dim3(256), 0, s, y, outMult, x, inMult, f, b, p, total);
  return check_launch("conv forward (direct)");
}

int conv_backward_data_direct(hipStream_t s, const ConvP& p, float* dx, float dxMult, const float* f, const float* dy) {
  const size_t total = (size_t)p.H * p.W * p.C * p.N;
  const size_t blocks = (total + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "conv backward-data: tensor too large");
  hipLaunchKernelGGL(conv_bwd_data_direct, dim3((unsigned)blocks), dim3(256), 0, s, dx, dxMult, f, dy, p, total);
  return check_launch("conv backward-data (direct)");
}

int conv_backward_filter_direct(hipStream_t s, const ConvP& p, float* df, const float* x, const float* dy) {
  const size_t total = (size_t)p.FH * p.FW * p.FC * p.K;
  if (total >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "conv backward-filter: filter bank too large");
  hipLaunchKernelGGL(conv_bwd_filter_direct, dim3((unsigned)total), dim3(256), 0, s, df, x, dy, p);
  return check_launch("conv backward-filter (direct)");
}

}  // namespace mcn
