// Double precision: the operators' VLDT_Double instantiation (matlab/src/bits/impl/dispatcher.hpp:60-98 switches on
// the tensors' data type; every operator of the path is instantiated for float and double, e.g.
// bits/nnconv.cu:444-469, bits/nnbnorm.cu:388-442, bits/nnpooling.cu:270-282).  These are the general kernels --
// one accumulator per output element, any geometry -- not tuned ones: the measured configurations are all single
// precision.  Results follow the reference's definitions; pooling keeps the order of its sequential loops, so its
// results have the same bits as the CPU reference (this file is compiled without floating-point contraction and
// uses fma() where a fused operation is meant).
#include "conv_common.hpp"

#include <algorithm>

namespace mcn {

bool pool_max_backward_stream_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, double* derInput,
                                     const double* x, const double* derOutput, int accumulate);  // pool_stream.hip
bool pool_avg_backward_tiles_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, double* derInput,
                                    const double* derOutput, int accumulate);  // pool.hip

namespace {

// ---------------------------------------------------------------------------------------------------------
// convolution (bits/nnconv.cu:71-317 with bits/impl/im2row_cpu.cpp:52-230 folded in)
// ---------------------------------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void conv64_forward(double* __restrict__ y, double outMult, const double* __restrict__ x,
                                                      double inMult, const double* __restrict__ f,
                                                      const double* __restrict__ b, ConvP p, size_t total) {
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
  const double* xn = x + (size_t)p.H * p.W * ((size_t)p.C * n + (size_t)g * p.FC);
  const double* fk = f + (size_t)p.FH * p.FW * p.FC * k;
  double acc = 0.0;
  for (int d = 0; d < p.FC; ++d)
    for (int j = 0; j < p.FW; ++j) {
      const int w = ow * p.sx + j * p.dx - p.pl;
      if ((unsigned)w >= (unsigned)p.W) continue;
      for (int i = 0; i < p.FH; ++i) {
        const int h = oh * p.sy + i * p.dy - p.pt;
        if ((unsigned)h >= (unsigned)p.H) continue;
        acc = fma(xn[h + p.H * (w + (size_t)p.W * d)], fk[i + p.FH * (j + p.FW * d)], acc);
      }
    }
  double r0 = inMult * acc;
  if (outMult != 0.0) r0 = fma(outMult, y[idx], r0);
  if (b) r0 += b[k];
  y[idx] = r0;
}

// UNIT: strides of 1 (every tap position is an output pixel: no divisions in the loops)
template <bool UNIT>
__global__ __launch_bounds__(256) void conv64_backward_data(double* __restrict__ dx, const double* __restrict__ f,
                                                            const double* __restrict__ dy, ConvP p, size_t total) {
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
  double acc = 0.0;
  for (int kk = 0; kk < p.Kg; ++kk) {
    const int k = g * p.Kg + kk;
    const double* dyk = dy + (size_t)P * ((size_t)p.K * n + k);
    const double* fk = f + (size_t)p.FH * p.FW * ((size_t)p.FC * k + d);
    for (int j = 0; j < p.FW; ++j) {
      const int aw = w + p.pl - j * p.dx;
      if (aw < 0 || (!UNIT && aw % p.sx)) continue;
      const int ow = UNIT ? aw : aw / p.sx;
      if (ow >= p.outW) continue;
      for (int i = 0; i < p.FH; ++i) {
        const int ah = h + p.pt - i * p.dy;
        if (ah < 0 || (!UNIT && ah % p.sy)) continue;
        const int oh = UNIT ? ah : ah / p.sy;
        if (oh >= p.outH) continue;
        acc = fma(dyk[oh + p.outH * ow], fk[i + p.FH * j], acc);
      }
    }
  }
  dx[idx] = acc;
}

// The same sums for a layer with at most four input channels (one filter group, strides and dilations of 1: a first
// layer): a thread owns one input pixel and all its channels, so a dzdy value is loaded once for all of them and the
// channels' sums are independent chains; the taps that land on an output pixel are a range worked out up front, so
// the loops carry no tests.  Each sum runs over (filter, column tap, row tap) ascending, as above: same bits.
// FHW > 0: a square window of that size, its loops unrolled -- the loads of a filter's whole window are in flight
// together, where the loops with run-time bounds (FHW == 0) wait for one load per turn.  A tap off the output
// contributes 0 * weight there (the reference adds nothing: the same unless that weight is not finite).
template <int CC, int FHW>
__global__ __launch_bounds__(256) void conv64_backward_data_few(double* __restrict__ dx, const double* __restrict__ f,
                                                                const double* __restrict__ dy, ConvP p, size_t pixels) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= pixels) return;
  const int FH = FHW > 0 ? FHW : p.FH, FW = FHW > 0 ? FHW : p.FW;
  const int HW = p.H * p.W, P = p.outH * p.outW, T = FH * FW;
  const size_t n = idx / HW;
  const int q = (int)(idx - n * HW);
  const int w = q / p.H, h = q - w * p.H;
  const int iLo = max(0, h + p.pt - (p.outH - 1)), iHi = min(FH - 1, h + p.pt);
  const int jLo = max(0, w + p.pl - (p.outW - 1)), jHi = min(FW - 1, w + p.pl);
  double acc[CC];
#pragma unroll
  for (int c = 0; c < CC; ++c) acc[c] = 0.0;
  const double* dy0 = dy + (size_t)P * p.K * n + (size_t)p.outH * (w + p.pl) + (h + p.pt);  // tap (0, 0) of filter 0
  if (FHW > 0) {
    // a tap that lands off the output reads the nearest tap that does not (a real value) and counts as zero: the loop
    // body is straight-line code (with a test per tap the compiler branches around every load and multiply)
    int rowOff[FHW > 0 ? FHW : 1], colOff[FHW > 0 ? FHW : 1];
#pragma unroll
    for (int i = 0; i < FHW; ++i) {
      rowOff[i] = -min(max(i, iLo), iHi);
      colOff[i] = -p.outH * min(max(i, jLo), jHi);
    }
#pragma unroll 2
    for (int k = 0; k < p.K; ++k) {
      const double* dyk = dy0 + (size_t)P * k;
      const double* fk = f + (size_t)T * CC * k;
      double v[FHW > 0 ? FHW : 1][FHW > 0 ? FHW : 1];
#pragma unroll
      for (int j = 0; j < FHW; ++j)
#pragma unroll
        for (int i = 0; i < FHW; ++i) {
          const double got = dyk[colOff[j] + rowOff[i]];
          v[j][i] = (j >= jLo && j <= jHi && i >= iLo && i <= iHi) ? got : 0.0;
        }
#pragma unroll
      for (int j = 0; j < FHW; ++j)
#pragma unroll
        for (int i = 0; i < FHW; ++i)
#pragma unroll
          for (int c = 0; c < CC; ++c) acc[c] = fma(v[j][i], fk[i + FHW * j + T * c], acc[c]);
    }
  } else {
    for (int k = 0; k < p.K; ++k) {
      const double* dyk = dy0 + (size_t)P * k;
      const double* fk = f + (size_t)T * CC * k;
      for (int j = jLo; j <= jHi; ++j)
        for (int i = iLo; i <= iHi; ++i) {
          const double v = dyk[-(p.outH * j + i)];
#pragma unroll
          for (int c = 0; c < CC; ++c) acc[c] = fma(v, fk[i + FH * j + T * c], acc[c]);
        }
    }
  }
#pragma unroll
  for (int c = 0; c < CC; ++c) dx[(size_t)q + (size_t)HW * (c + (size_t)CC * n)] = acc[c];
}

// sum of the four wavefronts' values, in a fixed order, on thread 0
__device__ __forceinline__ double block_sum(double v, double* lds) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  const double s = (lds[0] + lds[1]) + (lds[2] + lds[3]);
  __syncthreads();
  return s;
}

// sum of sixteen wavefronts' values, in a fixed order, on every thread
__device__ __forceinline__ double block_sum16(double v, double* lds) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  double s = 0.0;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += lds[i];
  __syncthreads();
  return s;
}

// one workgroup per filter element
__global__ __launch_bounds__(256) void conv64_backward_filter(double* __restrict__ df, const double* __restrict__ x,
                                                              const double* __restrict__ dy, ConvP p) {
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
      acc = fma(x[h + p.H * (w + (size_t)p.W * (c + (size_t)p.C * n))], dy[q + (size_t)P * (k + (size_t)p.K * n)], acc);
  }
  const double s = block_sum(acc, lds);
  if (threadIdx.x == 0) df[blockIdx.x] = s;
}

// one workgroup of sixteen wavefronts per filter: db[k] = sum over images and pixels of dy.  A thread walks the
// filter's N * P values 1024 apart -- (image, pixel) advanced by carries -- four at a time, so four loads are in
// flight per thread: with few filters the launch is a few workgroups, each of which has to keep its CU's memory path
// busy alone.
__global__ __launch_bounds__(1024) void conv64_backward_bias(double* __restrict__ db, const double* __restrict__ dy, int P,
                                                             int K, int N) {
  __shared__ double lds[16];
  const int k = blockIdx.x;
  if (P <= 0 || N <= 0) {  // (an empty output: the sum of nothing)
    if (threadIdx.x == 0) db[k] = 0.0;
    return;
  }
  const int stepN = 1024 / P, stepI = 1024 - stepN * P;  // 1024 values on: stepN images and stepI pixels
  int n = (int)threadIdx.x / P, i = (int)threadIdx.x - n * P;
  double a[4] = {0.0, 0.0, 0.0, 0.0};
  while (n < N) {
    double v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      v[u] = n < N ? dy[(size_t)P * (k + (size_t)K * n) + i] : 0.0;
      i += stepI;
      n += stepN;
      if (i >= P) {
        i -= P;
        ++n;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) a[u] += v[u];
  }
  const double s = block_sum16((a[0] + a[1]) + (a[2] + a[3]), lds);
  if (threadIdx.x == 0) db[k] = s;
}

// ---------------------------------------------------------------------------------------------------------
// The three products on the fp64 matrix instruction (groups == 1): C[m][n] = sum over k of A[m][k] B[k][n] with
//   forward          m = output pixel (all images), n = filter,        k = row of the filter volume;  A = the patch
//                    element (gathered from x, zero outside the image), B = the bank as stored
//   backward-data    m = input pixel,               n = input channel, k = (tap, filter);  A = dzdy where the tap of
//                    that filter lands on an output pixel (zero elsewhere), B = the bank read tap-major
//   backward-filter  m = row of the filter volume,  n = filter,        k = output pixel (all images), in splits;
//                    A = the patch element, B = dzdy; partial banks per split, added in split order afterwards
// v_mfma_f64_16x16x4_f64: lane l gives A[l % 16][l / 16] and B[l / 16][l % 16] and holds C[l / 16 + 4 i][l % 16],
// i = 0..3.  A workgroup makes a 64 x 64 tile (four wavefronts, 32 x 32 each: four accumulators) in stages of 16
// along k through LDS; the next stage's operands are fetched into registers while this one is multiplied.  A thread
// fetches four consecutive k of one m (and of one n): its m is decomposed once, its k once per stage and then by carries.
// ---------------------------------------------------------------------------------------------------------
typedef double doublex4 __attribute__((ext_vector_type(4)));

struct Gemm64P {
  ConvP c;
  int M, Nn, Kd;       // extents of the product
  int P, HW, FV, T;    // output pixels / input pixels of an image, rows of the filter volume, taps
  int chunk;           // backward-filter: k per split (a multiple of 16)
  double outMult, inMult;
  FastDiv byP, byOutH, byHW, byH, byFH, byT, bySy, bySx;
};

// FAST: strides and dilations of 1 and every tensor under 2^31 elements -- offsets are 32-bit sums of a part that
// depends on m (or n) alone and a part that depends on k alone, the latter advanced by carries; every load is issued
// (from offset 0 where its element does not exist) and what does not exist is zeroed afterwards, so the eight loads
// of a stage are in flight together.  (The general form spends 2.4 times the matrix instructions' cycles on 64-bit
// address arithmetic.)
template <int KIND, bool FAST>
__global__ __launch_bounds__(256, 2) void conv64_mfma(double* __restrict__ out, const double* __restrict__ a,
                                                      const double* __restrict__ b, const double* __restrict__ bias, Gemm64P p) {
  constexpr int KS = 16, LDA = KS + 1, LDB = 64 + 2;
  __shared__ double As[64 * LDA];
  __shared__ double Bs[KS * LDB];
  const ConvP& c = p.c;
  const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lk = lane >> 4;
  const int wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  const int kBegin = KIND == 2 ? blockIdx.z * p.chunk : 0;
  const int kEnd = KIND == 2 ? min(kBegin + p.chunk, p.Kd) : p.Kd;

  // ---- this thread's fetches: element (m0 + fm, k .. k + 3) of A and (k .. k + 3, n0 + fm) of B
  const int fm = tid & 63, fk = (tid >> 6) * 4;
  const int m = m0 + fm, n = n0 + fm;
  // what m means (fixed): KIND 0: output pixel; 1: input pixel; 2: row of the filter volume
  int mImg = 0, mH = 0, mW = 0, mC = 0;
  if (KIND == 0) {
    int q;
    p.byP.divmod(min(m, p.M - 1), &mImg, &q);
    p.byOutH.divmod(q, &mW, &mH);
  } else if (KIND == 1) {
    int e;
    p.byHW.divmod(min(m, p.M - 1), &mImg, &e);
    p.byH.divmod(e, &mW, &mH);
  } else {
    int t;
    p.byT.divmod(min(m, p.M - 1), &mC, &t);
    p.byFH.divmod(t, &mW, &mH);  // (mW, mH) = the tap (j, i)
  }
  double ra[4], rb[4];
  unsigned okMask = 0;  // FAST: bit u: ra[u] exists, bit 4 + u: rb[u] exists
  // FAST: the parts of the offsets that m and n fix
  int baseA = 0, baseB = 0;
  if (FAST) {
    if (KIND == 0) {
      baseA = (mH - c.pt) + c.H * ((mW - c.pl) + c.W * c.C * mImg);
      baseB = p.FV * min(n, p.Nn - 1);
    } else if (KIND == 1) {
      baseA = (mH + c.pt) + c.outH * ((mW + c.pl) + c.outW * c.K * mImg);
      baseB = p.T * min(n, p.Nn - 1);
    } else {
      baseA = (mH - c.pt) + c.H * ((mW - c.pl) + c.W * mC);
      baseB = p.P * min(n, p.Nn - 1);
    }
  }
  auto fetch = [&](int k0) {
    const int k = k0 + fk;
    if (FAST && (KIND == 0 || KIND == 1)) {
      int d, t, j, i;
      p.byT.divmod(k, &d, &t);
      p.byFH.divmod(t, &j, &i);
      // the parts that k fixes: KIND 0: x at (i, j, d) and the bank row k; KIND 1: dzdy at (-i, -j, d) and the bank
      // at (t, d)
      int offA = KIND == 0 ? i + c.H * (j + c.W * d) : p.P * d - c.outH * j - i;
      int offB = KIND == 0 ? k : t + p.T * c.C * d;
      const int rowStep = KIND == 0 ? c.H - c.FH : c.FH - c.outH;           // a column on, back to the first row
      const int volStep = KIND == 0 ? p.HW - c.H * c.FW : p.P + c.outH * c.FW;  // a channel (filter) on, back to the first column
      double la[4], lb[4];
      bool okA[4], okB[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int h = KIND == 0 ? mH - c.pt + i : mH + c.pt - i, w = KIND == 0 ? mW - c.pl + j : mW + c.pl - j;
        const bool inK = k + u < kEnd;
        okA[u] = inK && m < p.M && (unsigned)h < (unsigned)(KIND == 0 ? c.H : c.outH) &&
                 (unsigned)w < (unsigned)(KIND == 0 ? c.W : c.outW);
        okB[u] = inK && n < p.Nn;
        la[u] = a[okA[u] ? baseA + offA : 0];
        lb[u] = b[okB[u] ? baseB + offB : 0];
        offA += KIND == 0 ? 1 : -1;
        offB += 1;
        if (++i == c.FH) {
          i = 0;
          offA += rowStep;
          if (++j == c.FW) {
            j = 0;
            offA += volStep;
            if (KIND == 1) offB += p.T * c.C - p.T;
          }
        }
      }
      // (what does not exist is zeroed where the stage is written to LDS: a select here would wait for the loads
      // before this stage's matrix instructions)
      okMask = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        ra[u] = la[u];
        rb[u] = lb[u];
        okMask |= (okA[u] ? 1u : 0u) << u | (okB[u] ? 16u : 0u) << u;
      }
    } else if (FAST) {
      // k = output pixel of all images; x at (oh, ow, img) shifted by the tap, dzdy at pixel q of image img
      int img, q, ow, oh;
      p.byP.divmod(min(k, p.Kd - 1), &img, &q);
      p.byOutH.divmod(q, &ow, &oh);
      int offA = oh + c.H * ow + p.HW * c.C * img, offB = q + p.P * c.K * img;
      double la[4], lb[4];
      bool okA[4], okB[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int h = oh - c.pt + mH, w = ow - c.pl + mW;
        const bool inK = k + u < kEnd;
        okA[u] = inK && m < p.M && (unsigned)h < (unsigned)c.H && (unsigned)w < (unsigned)c.W;
        okB[u] = inK && n < p.Nn;
        la[u] = a[okA[u] ? baseA + offA : 0];
        lb[u] = b[okB[u] ? baseB + offB : 0];
        offA += 1;
        offB += 1;
        if (++oh == c.outH) {
          oh = 0;
          offA += c.H - c.outH;
          if (++ow == c.outW) {
            ow = 0;
            offA += p.HW * c.C - c.H * c.outW;
            offB += p.P * c.K - p.P;
          }
        }
      }
      // (what does not exist is zeroed where the stage is written to LDS: a select here would wait for the loads
      // before this stage's matrix instructions)
      okMask = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        ra[u] = la[u];
        rb[u] = lb[u];
        okMask |= (okA[u] ? 1u : 0u) << u | (okB[u] ? 16u : 0u) << u;
      }
    } else if (KIND == 0 || KIND == 1) {
      // k = t + T * (channel or filter), t = i + FH j
      int d, t, j, i;
      p.byT.divmod(k, &d, &t);
      p.byFH.divmod(t, &j, &i);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        double va = 0.0, vb = 0.0;
        if (k + u < kEnd) {
          if (KIND == 0) {
            const int h = mH * c.sy - c.pt + i * c.dy, w = mW * c.sx - c.pl + j * c.dx;
            if (m < p.M && (unsigned)h < (unsigned)c.H && (unsigned)w < (unsigned)c.W)
              va = a[h + (size_t)c.H * (w + (size_t)c.W * (d + (size_t)c.C * mImg))];
            if (n < p.Nn) vb = b[(size_t)(k + u) + (size_t)p.FV * n];
          } else {
            const int nh = mH + c.pt - i * c.dy, nw = mW + c.pl - j * c.dx;
            if (m < p.M && nh >= 0 && nw >= 0) {
              const int oh = p.bySy.div(nh), ow = p.bySx.div(nw);
              if (oh * c.sy == nh && ow * c.sx == nw && oh < c.outH && ow < c.outW)
                va = a[oh + (size_t)c.outH * (ow + (size_t)c.outW * (d + (size_t)c.K * mImg))];
            }
            if (n < p.Nn) vb = b[(size_t)t + (size_t)p.T * (n + (size_t)c.C * d)];
          }
        }
        ra[u] = va;
        rb[u] = vb;
        if (++i == c.FH) {
          i = 0;
          if (++j == c.FW) {
            j = 0;
            ++d;
          }
        }
        t = i + c.FH * j;
      }
    } else {
      // k = output pixel of all images
      int img, q, ow, oh;
      p.byP.divmod(min(k, p.Kd - 1), &img, &q);
      p.byOutH.divmod(q, &ow, &oh);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        double va = 0.0, vb = 0.0;
        if (k + u < kEnd) {
          const int h = oh * c.sy - c.pt + mH * c.dy, w = ow * c.sx - c.pl + mW * c.dx;
          if (m < p.M && (unsigned)h < (unsigned)c.H && (unsigned)w < (unsigned)c.W)
            va = a[h + (size_t)c.H * (w + (size_t)c.W * (mC + (size_t)c.C * img))];
          if (n < p.Nn) vb = b[oh + (size_t)c.outH * (ow + (size_t)c.outW * (n + (size_t)c.K * img))];
        }
        ra[u] = va;
        rb[u] = vb;
        if (++oh == c.outH) {
          oh = 0;
          if (++ow == c.outW) {
            ow = 0;
            ++img;
          }
        }
      }
    }
  };

  doublex4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (doublex4){0.0, 0.0, 0.0, 0.0};

  if (kBegin < kEnd) fetch(kBegin);
  for (int k0 = kBegin; k0 < kEnd; k0 += KS) {
    __syncthreads();  // (the stage before this one has been multiplied)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      As[fm * LDA + fk + u] = !FAST || (okMask >> u & 1u) ? ra[u] : 0.0;
      Bs[(fk + u) * LDB + fm] = !FAST || (okMask >> (4 + u) & 1u) ? rb[u] : 0.0;
    }
    __syncthreads();
    if (k0 + KS < kEnd) fetch(k0 + KS);
#pragma unroll
    for (int kk = 0; kk < KS / 4; ++kk) {
      double av[2], bv[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) av[i] = As[(32 * wm + 16 * i + l16) * LDA + 4 * kk + lk];
#pragma unroll
      for (int j = 0; j < 2; ++j) bv[j] = Bs[(4 * kk + lk) * LDB + 32 * wn + 16 * j + l16];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- element (row 32 wm + 16 i + lk + 4 e, column 32 wn + 16 j + l16) of the tile is acc[i][j][e]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int row = m0 + 32 * wm + 16 * i + lk + 4 * e, col = n0 + 32 * wn + 16 * j + l16;
        if (row >= p.M || col >= p.Nn) continue;
        const double v = acc[i][j][e];
        if (KIND == 0) {
          int img, q;
          p.byP.divmod(row, &img, &q);
          const size_t at = (size_t)q + (size_t)p.P * (col + (size_t)c.K * img);
          double r0 = p.inMult * v;
          if (p.outMult != 0.0) r0 = fma(p.outMult, out[at], r0);
          if (bias) r0 += bias[col];
          out[at] = r0;
        } else if (KIND == 1) {
          int img, el;
          p.byHW.divmod(row, &img, &el);
          out[(size_t)el + (size_t)p.HW * (col + (size_t)c.C * img)] = v;
        } else {
          // rows are t + T c here as in the bank (row = the stored index of the filter volume)
          out[(size_t)blockIdx.z * p.FV * c.K + (size_t)row + (size_t)p.FV * col] = v;
        }
      }
}

// dF[e] = sum over the splits' partial banks, in a fixed order: a workgroup owns 16 consecutive elements; thread
// (e, g) adds the splits g, g + 16, g + 32, ... (eight loads in flight), and the sixteen sums of an element are added
// in order of g.  (One thread per element walking all the splits waits for one load at a time: 256 splits of a
// 2400-element bank took 65 us that way.)
__global__ __launch_bounds__(256) void conv64_sum_splits(double* __restrict__ df, const double* __restrict__ partials, size_t n,
                                                         int splits) {
  __shared__ double part[16][17];
  const int le = threadIdx.x & 15, g = threadIdx.x >> 4;
  const size_t e = (size_t)blockIdx.x * 16 + le;
  double s = 0.0;
  if (e < n) {
    int i = g;
    for (; i + 112 < splits; i += 128) {
      double v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partials[(size_t)(i + 16 * u) * n + e];
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; i < splits; i += 16) s += partials[(size_t)i * n + e];
  }
  part[g][le] = s;
  __syncthreads();
  if (g == 0 && e < n) {
    double t = part[0][le];
#pragma unroll
    for (int k = 1; k < 16; ++k) t += part[k][le];
    df[e] = t;
  }
}

// ---------------------------------------------------------------------------------------------------------
// batch normalisation (bits/nnbnorm.cu:46-164: compute_moment, compute_ders, compute_ders_and_moments,
// batch_normalize_forward / _backward)
// ---------------------------------------------------------------------------------------------------------

// One workgroup of sixteen wavefronts per channel (a read-only stream: the more wavefronts a CU holds, the more loads
// are in flight).  DERS == false: sums of x and x*x, turned into (mean, sigma) in moments[c], moments[C + c].
// DERS == true: sums of dy and x*dy (and, unless the moments are given, of x and x*x as well); writes dzdb, dzdg and
// the moments.
template <bool DERS, bool GIVEN>
__global__ __launch_bounds__(1024) void bnorm64_sums(double* __restrict__ moments, double* __restrict__ dG,
                                                     double* __restrict__ dB, const double* __restrict__ x,
                                                     const double* __restrict__ dy, int WH, int C, int N, double epsilon) {
  __shared__ double lds[16];
  const int c = blockIdx.x;
  double sx = 0.0, sxx = 0.0, sd = 0.0, sxd = 0.0;
  for (int n = 0; n < N; ++n) {
    const size_t base = (size_t)WH * (c + (size_t)C * n);
    // (two elements per thread and turn: their loads are issued together)
    for (int i = threadIdx.x; i < WH; i += 2048) {
      const bool two = i + 1024 < WH;
      const double v0 = x[base + i], v1 = two ? x[base + i + 1024] : 0.0;
      double d0 = 0.0, d1 = 0.0;
      if (DERS) {
        d0 = dy[base + i];
        d1 = two ? dy[base + i + 1024] : 0.0;
      }
      if (!GIVEN) {
        sx += v0;
        sxx = fma(v0, v0, sxx);
        sx += v1;
        sxx = fma(v1, v1, sxx);
      }
      if (DERS) {
        sd += d0;
        sxd = fma(v0, d0, sxd);
        sd += d1;
        sxd = fma(v1, d1, sxd);
      }
    }
  }
  double mean, sigma;
  const double mass = (double)WH * (double)N;
  if (GIVEN) {
    mean = moments[c];
    sigma = moments[C + c];
  } else {
    sx = block_sum16(sx, lds);
    sxx = block_sum16(sxx, lds);
    mean = sx / mass;
    sigma = sqrt(fmax(0.0, sxx / mass - mean * mean) + epsilon);  // sigma includes epsilon (bits/nnbnorm.cu:65-70)
  }
  if (DERS) {
    sd = block_sum16(sd, lds);
    sxd = block_sum16(sxd, lds);
  }
  if (threadIdx.x != 0) return;
  if (!GIVEN) {
    moments[c] = mean;
    moments[C + c] = sigma;
  }
  if (DERS) {
    dB[c] = sd;
    dG[c] = (sxd - mean * sd) / sigma;  // bits/nnbnorm.cu:93-97,128-132
  }
}

// y = (g/sigma)*(x - mean) + b, rounded as written  (bits/nnbnorm.cu:192-203).  A workgroup works inside one plane
// (blockIdx.x = c + C n), on slab blockIdx.y of it: the channel's constants (two divisions) are worked out once per thread.
__global__ __launch_bounds__(256) void bnorm64_forward_apply(double* __restrict__ y, const double* __restrict__ x,
                                                             const double* __restrict__ moments,
                                                             const double* __restrict__ mult, const double* __restrict__ bias,
                                                             int WH, int C, int slab) {
  const int c = blockIdx.x % C;
  const double G = mult[c] / moments[C + c], mean = moments[c], b = bias[c];
  const size_t base = (size_t)blockIdx.x * WH;
  const int i0 = blockIdx.y * slab, i1 = min(i0 + slab, WH);
  for (int i = i0 + threadIdx.x; i < i1; i += 256) y[base + i] = G * (x[base + i] - mean) + b;
}

// dzdx = G1*(dzdy - dzdb/m) - G2*(x - mean),  G1 = g/sigma,  G2 = G1*dzdg/(m*sigma)  (bits/nnbnorm.cu:136-164)
__global__ __launch_bounds__(256) void bnorm64_backward_apply(double* __restrict__ dx, const double* __restrict__ x,
                                                              const double* __restrict__ dy,
                                                              const double* __restrict__ moments,
                                                              const double* __restrict__ mult, const double* __restrict__ dG,
                                                              const double* __restrict__ dB, int WH, int C, double mass,
                                                              int slab) {
  const int c = blockIdx.x % C;
  const double mean = moments[c], sigma = moments[C + c];
  const double muz = dB[c] / mass;
  const double G1 = mult[c] / sigma;
  const double G2 = G1 * dG[c] / (mass * sigma);
  const size_t base = (size_t)blockIdx.x * WH;
  const int i0 = blockIdx.y * slab, i1 = min(i0 + slab, WH);
  for (int i = i0 + threadIdx.x; i < i1; i += 256) dx[base + i] = G1 * (dy[base + i] - muz) - G2 * (x[base + i] - mean);
}

// ---------------------------------------------------------------------------------------------------------
// pooling (bits/nnpooling.cu:33-237)
// ---------------------------------------------------------------------------------------------------------

struct Pool64 {
  int H, W, outH, outW;
  int poolH, poolW, sy, sx, pt, pl;
  int accumulate;
};

// one thread per output: window clipped to the image, columns (slow) then rows (fast); max: first element greater
// than the running value, which starts at -inf (bits/nnpooling.cu:36-61); average: sum times T(1)/T(area) (:63-96)
template <bool MAX>
__global__ __launch_bounds__(256) void pool64_forward(double* __restrict__ y, const double* __restrict__ x, Pool64 p,
                                                      size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int P = p.outH * p.outW;
  const size_t plane = idx / P;
  const int q = (int)(idx - plane * P);
  const int ow = q / p.outH, oh = q - ow * p.outH;
  int h1 = oh * p.sy - p.pt, w1 = ow * p.sx - p.pl;
  const int h2 = min(h1 + p.poolH, p.H), w2 = min(w1 + p.poolW, p.W);
  h1 = max(h1, 0);
  w1 = max(w1, 0);
  const double* xp = x + plane * (size_t)p.H * p.W;
  if (MAX) {
    double best = -__builtin_inf();
    for (int w = w1; w < w2; ++w)
      for (int h = h1; h < h2; ++h) {
        const double v = xp[h + (size_t)p.H * w];
        if (v > best) best = v;
      }
    y[idx] = best;
  } else {
    double acc = 0.0;
    for (int w = w1; w < w2; ++w)
      for (int h = h1; h < h2; ++h) acc += xp[h + (size_t)p.H * w];
    y[idx] = acc * (1.0 / (double)((h2 - h1) * (w2 - w1)));
  }
}

// One thread per input element: the outputs whose window holds it, columns ascending then rows ascending -- the
// order in which the reference's loop over outputs adds to it (bits/nnpooling.cu:190-206) -- so the sum has the
// same bits.  Max: an output counts when this element is its window's winner (first maximum in memory order).
template <bool MAX>
__global__ __launch_bounds__(256) void pool64_backward(double* __restrict__ dx, const double* __restrict__ x,
                                                       const double* __restrict__ dy, Pool64 p, size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int HW = p.H * p.W;
  const size_t plane = idx / HW;
  const int e = (int)(idx - plane * HW);
  const int w = e / p.H, h = e - w * p.H;
  const double* xp = x ? x + plane * (size_t)HW : nullptr;
  const double* dyp = dy + plane * (size_t)p.outH * p.outW;
  // outputs o with o*s - pad <= h < o*s - pad + pool
  const int ohLo = max(0, (h + p.pt - p.poolH + p.sy) / p.sy), ohHi = min(p.outH - 1, (h + p.pt) / p.sy);
  const int owLo = max(0, (w + p.pl - p.poolW + p.sx) / p.sx), owHi = min(p.outW - 1, (w + p.pl) / p.sx);
  double acc = p.accumulate ? dx[idx] : 0.0;
  for (int ow = owLo; ow <= owHi; ++ow)
    for (int oh = ohLo; oh <= ohHi; ++oh) {
      int h1 = oh * p.sy - p.pt, w1 = ow * p.sx - p.pl;
      const int h2 = min(h1 + p.poolH, p.H), w2 = min(w1 + p.poolW, p.W);
      h1 = max(h1, 0);
      w1 = max(w1, 0);
      if (h < h1 || h >= h2 || w < w1 || w >= w2) continue;
      const double d = dyp[oh + (size_t)p.outH * ow];
      if (MAX) {
        double best = -__builtin_inf();
        int at = -1;
        for (int ww = w1; ww < w2; ++ww)
          for (int hh = h1; hh < h2; ++hh) {
            const double v = xp[hh + (size_t)p.H * ww];
            if (v > best) {
              best = v;
              at = hh + p.H * ww;
            }
          }
        if (at == e) acc += d;
      } else {
        acc += d * (1.0 / (double)((h2 - h1) * (w2 - w1)));
      }
    }
  dx[idx] = acc;
}

// The same sums by tiles through LDS (max only; the kernel above reads each window once per element it holds, from the
// caches).  A workgroup owns a strip of input columns of one plane: it stages the strip's x with the columns its
// outputs' windows reach, and those outputs' dzdy; finds every such output's winner once (the same search); then each
// thread adds, for an element of the strip, the dzdy of the outputs that chose it, in the same order as above -- so
// the same bits.
struct Pool64Tile {
  int TW;          // input columns of a strip
  int maxXW, maxOW;  // most x columns / output columns a strip stages
  int items;                             // strips of all planes
  int rowsIn, colsIn, rowsOut, colsOut;  // threads as rows x columns: of the strip's inputs, of its outputs
  FastDiv byRowsIn, byRowsOut, bySy, bySx;
};

// what strip `strip` stages: its owned columns [w0, w1), the outputs [owLo, owLo + nOW) and x columns [xLo, xLo + nXW)
struct Pool64Strip { int w0, w1, owLo, nOW, xLo, nXW; };
__host__ __device__ inline Pool64Strip pool64_strip(const Pool64& p, int TW, int strip) {
  Pool64Strip s;
  s.w0 = strip * TW;
  s.w1 = s.w0 + TW < p.W ? s.w0 + TW : p.W;
  int lo = (s.w0 + p.pl - p.poolW + p.sx) / p.sx, hi = (s.w1 - 1 + p.pl) / p.sx;
  lo = lo > 0 ? lo : 0;
  hi = hi < p.outW - 1 ? hi : p.outW - 1;
  s.owLo = lo;
  s.nOW = hi >= lo ? hi - lo + 1 : 0;
  int xLo = s.w0, xHi = s.w1;
  if (s.nOW > 0) {
    xLo = xLo < lo * p.sx - p.pl ? xLo : lo * p.sx - p.pl;
    xHi = xHi > hi * p.sx - p.pl + p.poolW ? xHi : hi * p.sx - p.pl + p.poolW;
  }
  xLo = xLo > 0 ? xLo : 0;
  xHi = xHi < p.W ? xHi : p.W;
  s.xLo = xLo;
  s.nXW = xHi - xLo;
  return s;
}

// PH, PW, SY, SX > 0: the window and stride are these constants, and the loops over a window / over the outputs that hold
// an element are unrolled with predicates (same order of comparisons and sums): their LDS reads are independent and
// in flight together, where the loops with run-time bounds wait for one read per turn.  0: any geometry.
template <int PH, int PW, int SY, int SX>
__global__ __launch_bounds__(256) void pool64_max_backward_tiled(double* __restrict__ dx, const double* __restrict__ x,
                                                                 const double* __restrict__ dy, Pool64 p, Pool64Tile t,
                                                                 int strips) {
  extern __shared__ double tile[];
  const int tid = threadIdx.x;
  double* xs = tile;                                    // [nXW][H]
  double* ds = tile + (size_t)t.maxXW * p.H;            // [nOW][outH]
  int* win = (int*)(ds + (size_t)t.maxOW * p.outH);     // [nOW][outH]: the winner's index in the plane
  const size_t HW = (size_t)p.H * p.W;
  // A workgroup walks strips blockIdx.x, blockIdx.x + gridDim.x, ...: the next strip's loads (up to twelve of x and
  // four of dzdy per thread, into registers) are in flight while this strip is worked on.
  double vx[12], vd[4];
  auto fetch = [&](int item) {
    const int plane = item / strips;
    const Pool64Strip st = pool64_strip(p, t.TW, item - plane * strips);
    const double* xp = x + (size_t)plane * HW + (size_t)st.xLo * p.H;
    const double* dyp = dy + (size_t)plane * p.outH * p.outW + (size_t)st.owLo * p.outH;
    const int nX = st.nXW * p.H, nD = st.nOW * p.outH;
#pragma unroll
    for (int u = 0; u < 12; ++u) vx[u] = tid + u * 256 < nX ? xp[tid + u * 256] : 0.0;
#pragma unroll
    for (int u = 0; u < 4; ++u) vd[u] = tid + u * 256 < nD ? dyp[tid + u * 256] : 0.0;
  };
  int item = blockIdx.x;
  if (item < t.items) fetch(item);
  for (; item < t.items; item += gridDim.x) {
  const int plane = item / strips, strip = item - plane * strips;
  // owned columns, the outputs whose window holds one of them, and the x columns those windows reach
  const Pool64Strip st = pool64_strip(p, t.TW, strip);
  const int w0 = st.w0, w1 = st.w1, owLo = st.owLo, nOW = st.nOW, xLo = st.xLo, nXW = st.nXW;
  __syncthreads();  // (the strip before this one is done with the tile)
  {
    const int nX = nXW * p.H, nD = nOW * p.outH;
#pragma unroll
    for (int u = 0; u < 12; ++u)
      if (tid + u * 256 < nX) xs[tid + u * 256] = vx[u];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (tid + u * 256 < nD) ds[tid + u * 256] = vd[u];
  }
  __syncthreads();
  if (item + (int)gridDim.x < t.items) fetch(item + gridDim.x);
  // ---- winners: a thread keeps its output row and walks the strip's output columns (the row bounds of its windows
  // are worked out once)
  {
    int cq, oh;
    t.byRowsOut.divmod(tid, &cq, &oh);
    if (cq < t.colsOut) {
      for (; oh < p.outH; oh += t.rowsOut) {
        int h1 = oh * p.sy - p.pt;
        const int h2 = min(h1 + p.poolH, p.H);
        h1 = max(h1, 0);
        for (int o = cq; o < nOW; o += t.colsOut) {
          const int ow = owLo + o;
          int c1 = ow * p.sx - p.pl;
          const int c2 = min(c1 + p.poolW, p.W);
          c1 = max(c1, 0);
          double best = -__builtin_inf();
          int at = -1;
          if (PH > 0) {
            const int hr = oh * SY - p.pt, cr = ow * SX - p.pl;  // the window before clipping
            double v[PW > 0 ? PW : 1][PH > 0 ? PH : 1];
#pragma unroll
            for (int b = 0; b < PW; ++b)
#pragma unroll
              for (int a = 0; a < PH; ++a)
                v[b][a] = xs[min(max(hr + a, 0), p.H - 1) + p.H * (min(max(cr + b, xLo), xLo + nXW - 1) - xLo)];
#pragma unroll
            for (int b = 0; b < PW; ++b)
#pragma unroll
              for (int a = 0; a < PH; ++a) {
                const bool in = hr + a >= h1 && hr + a < h2 && cr + b >= c1 && cr + b < c2;
                if (in && v[b][a] > best) {
                  best = v[b][a];
                  at = hr + a + p.H * (cr + b);
                }
              }
          } else {
            for (int ww = c1; ww < c2; ++ww) {
              const double* col = xs + p.H * (ww - xLo);
              for (int hh = h1; hh < h2; ++hh) {
                const double v = col[hh];
                if (v > best) {
                  best = v;
                  at = hh + p.H * ww;
                }
              }
            }
          }
          win[oh + p.outH * o] = at;
        }
      }
    }
  }
  __syncthreads();
  // ---- sums: a thread keeps its input row (the output rows whose windows hold it: once) and walks the strip's columns
  {
    int cq, h;
    t.byRowsIn.divmod(tid, &cq, &h);
    if (cq < t.colsIn) {
      double* dxp = dx + (size_t)plane * HW + (size_t)w0 * p.H;
      for (; h < p.H; h += t.rowsIn) {
        // (a negative numerator can only give a first output below 0, which is clipped to 0 anyway)
        const int nh = h + p.pt - p.poolH + p.sy;
        const int ohLo = nh > 0 ? t.bySy.div(nh) : 0, ohHi = min(p.outH - 1, t.bySy.div(h + p.pt));
        for (int c = cq; c < w1 - w0; c += t.colsIn) {
          const int w = w0 + c, e = h + p.H * w;
          const int nw = w + p.pl - p.poolW + p.sx;
          const int oLo = nw > 0 ? t.bySx.div(nw) : 0, oHi = min(p.outW - 1, t.bySx.div(w + p.pl));
          double acc = p.accumulate ? dxp[h + p.H * c] : 0.0;
          if (PH > 0) {
            constexpr int NR = PH > 0 ? (PH + SY - 1) / (SY > 0 ? SY : 1) : 1, NC = PW > 0 ? (PW + SX - 1) / (SX > 0 ? SX : 1) : 1;
            int wn[NC][NR];
            double dv[NC][NR];
#pragma unroll
            for (int b = 0; b < NC; ++b)
#pragma unroll
              for (int a = 0; a < NR; ++a) {
                const int j = min(ohLo + a, p.outH - 1) + p.outH * (min(oLo + b, owLo + nOW - 1) - owLo);
                wn[b][a] = win[j];
                dv[b][a] = ds[j];
              }
#pragma unroll
            for (int b = 0; b < NC; ++b)
#pragma unroll
              for (int a = 0; a < NR; ++a)
                if (oLo + b <= oHi && ohLo + a <= ohHi && wn[b][a] == e) acc += dv[b][a];
          } else {
            for (int ow = oLo; ow <= oHi; ++ow)
              for (int oh = ohLo; oh <= ohHi; ++oh) {
                // (the window holds the element: the bounds above are exact for a window clipped to the image)
                const int j = oh + p.outH * (ow - owLo);
                if (win[j] == e) acc += ds[j];
              }
          }
          dxp[h + p.H * c] = acc;
        }
      }
    }
  }
  }  // (strips of this workgroup)
}

// The matrix-instruction form of a product (kind 0 forward, 1 backward-data, 2 backward-filter): one filter group,
// every extent inside 31 bits, and at least sixteen columns of the product (fewer: the one-accumulator kernels above
// multiply nothing in vain, a 64-wide tile would).
// unit strides and dilations, every tensor under 2^31 elements: the matrix kernels' 32-bit offsets (FAST)
bool gemm64_fast(const ConvP& c) {
  const long long lim = 1ll << 31;
  return c.sy == 1 && c.sx == 1 && c.dy == 1 && c.dx == 1 && (long long)c.H * c.W * c.C * c.N < lim &&
         (long long)c.outH * c.outW * c.K * c.N < lim && (long long)c.FH * c.FW * c.FC * c.K < lim;
}

bool gemm64_plan(const ConvP& c, int kind, Gemm64P* out) {
  if (c.groups != 1 || tunable("conv64_no_mfma", 0)) return false;
  const long long P = (long long)c.outH * c.outW, HW = (long long)c.H * c.W, T = (long long)c.FH * c.FW, FV = T * c.C;
  const long long M = kind == 0 ? P * c.N : (kind == 1 ? HW * c.N : FV);
  const long long Nn = kind == 1 ? c.C : c.K;
  const long long Kd = kind == 0 ? FV : (kind == 1 ? T * c.K : P * c.N);
  if (M < 1 || Nn < 16 || Kd < 1 || M >= (1ll << 30) || Kd >= (1ll << 30) || FV >= (1ll << 30) || (M + 63) / 64 >= (1ll << 31) ||
      (Nn + 63) / 64 > 65535)
    return false;
  Gemm64P p;
  p.c = c;
  p.M = (int)M; p.Nn = (int)Nn; p.Kd = (int)Kd;
  p.P = (int)P; p.HW = (int)HW; p.FV = (int)FV; p.T = (int)T;
  p.chunk = (int)Kd;
  p.outMult = 0.0;
  p.inMult = 1.0;
  p.byP = FastDiv((int)std::max(1ll, P)); p.byOutH = FastDiv(std::max(1, c.outH)); p.byHW = FastDiv((int)std::max(1ll, HW));
  p.byH = FastDiv(std::max(1, c.H)); p.byFH = FastDiv(c.FH); p.byT = FastDiv((int)T); p.bySy = FastDiv(c.sy); p.bySx = FastDiv(c.sx);
  *out = p;
  return true;
}

// the grid of the apply passes: planes x slabs of a plane (1024 elements, or more where a plane has over 65535 of them)
int plane_slabs(int WH, int C, int N, const char* who, int* slab, int* slabs) {
  if ((long long)C * N >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
  int sl = 1024;
  while ((WH + sl - 1) / sl > 65535) sl *= 2;
  *slab = sl;
  *slabs = (WH + sl - 1) / sl;
  return MCN_SUCCESS;
}

int blocks_for(size_t total, const char* who, unsigned* blocks) {
  const size_t b = (total + 255) / 256;
  if (b >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
  *blocks = (unsigned)b;
  return MCN_SUCCESS;
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

int mcn_conv_forward_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* y, double outMult, const double* x,
                         double inMult, const double* filters, const double* bias) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_forward_f64", &p);
  if (rc) return rc;
  const size_t total = (size_t)p.outH * p.outW * p.K * p.N;
  if (total == 0) return MCN_SUCCESS;
  if (!y || !x || !filters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_forward_f64: null tensor");
  Gemm64P gp;
  if (gemm64_plan(p, 0, &gp)) {
    gp.outMult = outMult;
    gp.inMult = inMult;
    KernelTimer timer("conv64_mfma", as_stream(stream));
    const dim3 grid((unsigned)((gp.M + 63) / 64), (unsigned)((gp.Nn + 63) / 64));
    if (gemm64_fast(p)) hipLaunchKernelGGL((conv64_mfma<0, true>), grid, dim3(256), 0, as_stream(stream), y, x, filters, bias, gp);
    else hipLaunchKernelGGL((conv64_mfma<0, false>), grid, dim3(256), 0, as_stream(stream), y, x, filters, bias, gp);
    return check_launch("mcn_conv_forward_f64");
  }
  unsigned blocks;
  if ((rc = blocks_for(total, "mcn_conv_forward_f64", &blocks))) return rc;
  KernelTimer timer("conv64_forward", as_stream(stream));
  hipLaunchKernelGGL(conv64_forward, dim3(blocks), dim3(256), 0, as_stream(stream), y, outMult, x, inMult, filters, bias, p,
                     total);
  return check_launch("mcn_conv_forward_f64");
}

int mcn_conv_backward_data_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derInput, const double* filters,
                               const double* derOutput) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_data_f64", &p);
  if (rc) return rc;
  const size_t total = (size_t)p.H * p.W * p.C * p.N;
  if (total == 0) return MCN_SUCCESS;
  if (!derInput || !filters || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_data_f64: null tensor");
  Gemm64P gp;
  if (gemm64_plan(p, 1, &gp)) {
    KernelTimer timer("conv64_mfma", as_stream(stream));
    const dim3 grid((unsigned)((gp.M + 63) / 64), (unsigned)((gp.Nn + 63) / 64));
    if (gemm64_fast(p))
      hipLaunchKernelGGL((conv64_mfma<1, true>), grid, dim3(256), 0, as_stream(stream), derInput, derOutput, filters, nullptr, gp);
    else
      hipLaunchKernelGGL((conv64_mfma<1, false>), grid, dim3(256), 0, as_stream(stream), derInput, derOutput, filters, nullptr, gp);
    return check_launch("mcn_conv_backward_data_f64");
  }
  unsigned blocks;
  if (p.groups == 1 && p.C <= 4 && p.sy == 1 && p.sx == 1 && p.dy == 1 && p.dx == 1 && !tunable("conv64_no_mfma", 0)) {
    const size_t pixels = total / p.C;
    if ((rc = blocks_for(pixels, "mcn_conv_backward_data_f64", &blocks))) return rc;
    KernelTimer timer("conv64_backward_data_few", as_stream(stream));
    hipStream_t st = as_stream(stream);
    const int sq = p.FH == p.FW && (p.FH == 3 || p.FH == 5 || p.FH == 7) ? p.FH : 0;
#define MCN_FEW64(CCF, FHF) \
  hipLaunchKernelGGL((conv64_backward_data_few<CCF, FHF>), dim3(blocks), dim3(256), 0, st, derInput, filters, derOutput, p, pixels)
#define MCN_FEW64_C(FHF)            \
  do {                              \
    if (p.C == 1) MCN_FEW64(1, FHF); \
    else if (p.C == 2) MCN_FEW64(2, FHF); \
    else if (p.C == 3) MCN_FEW64(3, FHF); \
    else MCN_FEW64(4, FHF);          \
  } while (0)
    if (sq == 3) MCN_FEW64_C(3);
    else if (sq == 5) MCN_FEW64_C(5);
    else if (sq == 7) MCN_FEW64_C(7);
    else MCN_FEW64_C(0);
#undef MCN_FEW64_C
#undef MCN_FEW64
    return check_launch("mcn_conv_backward_data_f64");
  }
  if ((rc = blocks_for(total, "mcn_conv_backward_data_f64", &blocks))) return rc;
  KernelTimer timer("conv64_backward_data", as_stream(stream));
  if (p.sy == 1 && p.sx == 1)
    hipLaunchKernelGGL(conv64_backward_data<true>, dim3(blocks), dim3(256), 0, as_stream(stream), derInput, filters, derOutput,
                       p, total);
  else
    hipLaunchKernelGGL(conv64_backward_data<false>, dim3(blocks), dim3(256), 0, as_stream(stream), derInput, filters, derOutput,
                       p, total);
  return check_launch("mcn_conv_backward_data_f64");
}

int mcn_conv_backward_filter_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derFilters, const double* x,
                                 const double* derOutput) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_filter_f64", &p);
  if (rc) return rc;
  if (!derFilters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_f64: null tensor");
  const size_t total = (size_t)p.FH * p.FW * p.FC * p.K;
  if ((size_t)p.outH * p.outW * p.N != 0 && (!x || !derOutput))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_f64: null tensor");
  Gemm64P gp;
  if ((size_t)p.outH * p.outW * p.N != 0 && gemm64_plan(p, 2, &gp) && gp.M >= 16) {
    // the pixels in splits, so that the launch fills the chip about twice; the partial banks live in memory taken from
    // (and given back to) the stream's pool
    hipStream_t st = as_stream(stream);
    int cus = device_compute_units();
    if (cus <= 0) cus = 256;
    const long long tiles = (long long)((gp.M + 63) / 64) * ((gp.Nn + 63) / 64);
    long long splits = std::max(1ll, std::min<long long>((2ll * cus + tiles - 1) / tiles, (gp.Kd + 255) / 256));
    splits = std::min(splits, 65535ll);
    gp.chunk = (int)(((gp.Kd + splits - 1) / splits + 15) / 16 * 16);
    splits = (gp.Kd + gp.chunk - 1) / gp.chunk;
    void* partials = nullptr;
    if (splits > 1 && hipMallocAsync(&partials, (size_t)splits * total * sizeof(double), st) != hipSuccess) {
      (void)hipGetLastError();
      partials = nullptr;
      splits = 1;
      gp.chunk = gp.Kd;
    }
    {
      KernelTimer timer("conv64_mfma", st);
      const dim3 grid((unsigned)((gp.M + 63) / 64), (unsigned)((gp.Nn + 63) / 64), (unsigned)splits);
      double* target = splits > 1 ? (double*)partials : derFilters;
      if (gemm64_fast(p)) hipLaunchKernelGGL((conv64_mfma<2, true>), grid, dim3(256), 0, st, target, x, derOutput, nullptr, gp);
      else hipLaunchKernelGGL((conv64_mfma<2, false>), grid, dim3(256), 0, st, target, x, derOutput, nullptr, gp);
    }
    rc = check_launch("mcn_conv_backward_filter_f64");
    if (splits > 1) {
      if (!rc) {
        KernelTimer timer("conv64_sum_splits", st);
        hipLaunchKernelGGL(conv64_sum_splits, dim3((unsigned)((total + 15) / 16)), dim3(256), 0, st, derFilters,
                           (const double*)partials, total, (int)splits);
        rc = check_launch("mcn_conv_backward_filter_f64");
      }
      if (hipFreeAsync(partials, st) != hipSuccess) (void)hipGetLastError();
    }
    return rc;
  }
  KernelTimer timer("conv64_backward_filter", as_stream(stream));
  hipLaunchKernelGGL(conv64_backward_filter, dim3((unsigned)total), dim3(256), 0, as_stream(stream), derFilters, x, derOutput,
                     p);
  return check_launch("mcn_conv_backward_filter_f64");
}

int mcn_conv_backward_bias_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derBias, const double* derOutput) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_bias_f64", &p);
  if (rc) return rc;
  if (!derBias) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_bias_f64: null tensor");
  if ((size_t)p.outH * p.outW * p.N != 0 && !derOutput)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_bias_f64: null tensor");
  KernelTimer timer("conv64_backward_bias", as_stream(stream));
  hipLaunchKernelGGL(conv64_backward_bias, dim3((unsigned)p.K), dim3(1024), 0, as_stream(stream), derBias, derOutput,
                     p.outH * p.outW, p.K, p.N);
  return check_launch("mcn_conv_backward_bias_f64");
}

int mcn_bnorm_forward_f64(mcn_stream_t stream, double* y, double* moments, const double* x, const double* multipliers,
                          const double* biases, int H, int W, int C, int N, double epsilon, int givenMoments,
                          void* workspace, size_t workspaceBytes) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward_f64: negative tensor extent");
  if ((long long)H * W >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "mcn_bnorm_forward_f64: plane too large");
  const size_t total = (size_t)H * W * C * N;
  if (C == 0) return MCN_SUCCESS;
  if ((total != 0 && (!y || !x)) || !multipliers || !biases) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward_f64: null tensor");
  if (givenMoments && !moments) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward_f64: MOMENTS are required when given");
  double* mom = moments;
  if (!mom) {
    if (!workspace || workspaceBytes < (size_t)2 * C * sizeof(double))
      return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward_f64: workspace too small (%zu < %zu bytes)", workspaceBytes,
                  (size_t)2 * C * sizeof(double));
    mom = (double*)workspace;
  }
  hipStream_t s = as_stream(stream);
  if (!givenMoments) {
    KernelTimer timer("bnorm64_sums", s);
    hipLaunchKernelGGL((bnorm64_sums<false, false>), dim3((unsigned)C), dim3(1024), 0, s, mom, nullptr, nullptr, x, nullptr,
                       H * W, C, N, epsilon);
    int rc = check_launch("mcn_bnorm_forward_f64");
    if (rc) return rc;
  }
  if (total == 0) return MCN_SUCCESS;
  int slab, slabs;
  int rc = plane_slabs(H * W, C, N, "mcn_bnorm_forward_f64", &slab, &slabs);
  if (rc) return rc;
  KernelTimer timer("bnorm64_forward_apply", s);
  hipLaunchKernelGGL(bnorm64_forward_apply, dim3((unsigned)(C * N), (unsigned)slabs), dim3(256), 0, s, y, x, mom, multipliers,
                     biases, H * W, C, slab);
  return check_launch("mcn_bnorm_forward_f64");
}

int mcn_bnorm_backward_f64(mcn_stream_t stream, double* derInput, double* derMultipliers, double* derBiases, double* moments,
                           const double* x, const double* multipliers, const double* derOutput, int H, int W, int C, int N,
                           double epsilon, int givenMoments, void* workspace, size_t workspaceBytes) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_f64: negative tensor extent");
  if ((long long)H * W >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "mcn_bnorm_backward_f64: plane too large");
  const size_t total = (size_t)H * W * C * N;
  if (C == 0) return MCN_SUCCESS;
  if ((total != 0 && (!derInput || !x || !derOutput)) || !multipliers || !derMultipliers || !derBiases)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_f64: null tensor");
  if (givenMoments && !moments) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_f64: MOMENTS are required when given");
  double* mom = moments;
  if (!mom) {
    if (!workspace || workspaceBytes < (size_t)2 * C * sizeof(double))
      return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_f64: workspace too small (%zu < %zu bytes)", workspaceBytes,
                  (size_t)2 * C * sizeof(double));
    mom = (double*)workspace;
  }
  hipStream_t s = as_stream(stream);
  {
    KernelTimer timer("bnorm64_sums", s);
    if (givenMoments)
      hipLaunchKernelGGL((bnorm64_sums<true, true>), dim3((unsigned)C), dim3(1024), 0, s, mom, derMultipliers, derBiases, x,
                         derOutput, H * W, C, N, epsilon);
    else
      hipLaunchKernelGGL((bnorm64_sums<true, false>), dim3((unsigned)C), dim3(1024), 0, s, mom, derMultipliers, derBiases, x,
                         derOutput, H * W, C, N, epsilon);
    int rc = check_launch("mcn_bnorm_backward_f64");
    if (rc) return rc;
  }
  if (total == 0) return MCN_SUCCESS;
  int slab, slabs;
  int rc = plane_slabs(H * W, C, N, "mcn_bnorm_backward_f64", &slab, &slabs);
  if (rc) return rc;
  KernelTimer timer("bnorm64_backward_apply", s);
  hipLaunchKernelGGL(bnorm64_backward_apply, dim3((unsigned)(C * N), (unsigned)slabs), dim3(256), 0, s, derInput, x, derOutput,
                     mom, multipliers, derMultipliers, derBiases, H * W, C, (double)H * W * (double)N, slab);
  return check_launch("mcn_bnorm_backward_f64");
}

int mcn_pool_forward_f64(mcn_stream_t stream, const mcn_pool_geom* g, double* y, const double* x) {
  int oh = 0, ow = 0;
  int rc = mcn_pool_output_size(g, &oh, &ow);
  if (rc) return rc;
  const size_t total = (size_t)oh * ow * g->C * g->N;
  if (total == 0) return MCN_SUCCESS;
  if (!y || !x) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_pool_forward_f64: null tensor");
  Pool64 p = {g->H, g->W, oh, ow, g->poolH, g->poolW, g->strideY, g->strideX, g->padTop, g->padLeft, 0};
  unsigned blocks;
  if ((rc = blocks_for(total, "mcn_pool_forward_f64", &blocks))) return rc;
  KernelTimer timer("pool64_forward", as_stream(stream));
  if (g->method == MCN_POOL_MAX)
    hipLaunchKernelGGL(pool64_forward<true>, dim3(blocks), dim3(256), 0, as_stream(stream), y, x, p, total);
  else
    hipLaunchKernelGGL(pool64_forward<false>, dim3(blocks), dim3(256), 0, as_stream(stream), y, x, p, total);
  return check_launch("mcn_pool_forward_f64");
}

int mcn_pool_backward_f64(mcn_stream_t stream, const mcn_pool_geom* g, double* derInput, const double* x,
                          const double* derOutput, int accumulate) {
  int oh = 0, ow = 0;
  int rc = mcn_pool_output_size(g, &oh, &ow);
  if (rc) return rc;
  const size_t total = (size_t)g->H * g->W * g->C * g->N;
  if (total == 0) return MCN_SUCCESS;
  const bool isMax = g->method == MCN_POOL_MAX;
  if (!derInput || !derOutput || (isMax && !x)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_pool_backward_f64: null tensor");
  Pool64 p = {g->H, g->W, oh, ow, g->poolH, g->poolW, g->strideY, g->strideX, g->padTop, g->padLeft, accumulate ? 1 : 0};
  unsigned blocks;
  if ((rc = blocks_for(total, "mcn_pool_backward_f64", &blocks))) return rc;
  // the streaming kernel of single precision, for the shapes it takes (columns of whole 16-byte cells, windows over at
  // most 2 x 2 outputs); same bits as the kernels below
  if (isMax && !tunable("pool64_no_tiles", 0) &&
      pool_max_backward_stream_launch(as_stream(stream), g, oh, ow, derInput, x, derOutput, accumulate))
    return check_launch("mcn_pool_backward_f64");
  // averages over windows that tile the plane exactly: single precision's streaming pass in memory order
  if (!isMax && !tunable("pool64_no_tiles", 0) &&
      pool_avg_backward_tiles_launch(as_stream(stream), g, oh, ow, derInput, derOutput, accumulate))
    return check_launch("mcn_pool_backward_f64");
  if (isMax && !tunable("pool64_no_tiles", 0)) {
    // strips of input columns through LDS, when a strip with its halo fits
    const int sx = g->strideX, sy = g->strideY;
    for (int TW = 32; TW >= 4; TW /= 2) {
      const int tw = std::min(TW, g->W);
      const int nStrips = (g->W + tw - 1) / tw;
      int maxOW = 1, maxXW = 1;
      for (int i = 0; i < nStrips; ++i) {
        const Pool64Strip st = pool64_strip(p, tw, i);
        maxOW = std::max(maxOW, st.nOW);
        maxXW = std::max(maxXW, st.nXW);
      }
      const size_t bytes = ((size_t)maxXW * g->H + (size_t)maxOW * oh) * sizeof(double) + (size_t)maxOW * oh * sizeof(int);
      const long long strips = (g->W + tw - 1) / tw, wgs = strips * (long long)g->C * g->N;
      // (a strip is fetched into registers one strip ahead: twelve x values and four of dzdy per thread at most)
      if (bytes > (size_t)40 * 1024 || wgs >= (1ll << 31) || sy < 1 || sx < 1 ||
          (long long)maxXW * g->H > 12 * 256 || (long long)maxOW * oh > 4 * 256)
        continue;
      Pool64Tile t;
      t.TW = tw;
      t.maxXW = maxXW;
      t.maxOW = maxOW;
      t.rowsIn = std::min(g->H, 256);
      t.colsIn = 256 / t.rowsIn;
      t.rowsOut = std::min(oh, 256);
      t.colsOut = 256 / t.rowsOut;
      t.byRowsIn = FastDiv(t.rowsIn);
      t.byRowsOut = FastDiv(t.rowsOut);
      t.bySy = FastDiv(sy);
      t.bySx = FastDiv(sx);
      KernelTimer timer("pool64_max_backward_tiled", as_stream(stream));
      t.items = (int)wgs;
      // (one strip per workgroup: resident workgroups walking the strips with the next strip's loads in flight
      // measured slower, 36.7 against 32.6 us on 112x112x64x8; the kernel's loop serves either launch)
      const dim3 grid((unsigned)wgs), block(256);
      hipStream_t st = as_stream(stream);
      if (g->poolH == 3 && g->poolW == 3 && sy == 2 && sx == 2)
        hipLaunchKernelGGL((pool64_max_backward_tiled<3, 3, 2, 2>), grid, block, bytes, st, derInput, x, derOutput, p, t, (int)strips);
      else if (g->poolH == 2 && g->poolW == 2 && sy == 2 && sx == 2)
        hipLaunchKernelGGL((pool64_max_backward_tiled<2, 2, 2, 2>), grid, block, bytes, st, derInput, x, derOutput, p, t, (int)strips);
      else
        hipLaunchKernelGGL((pool64_max_backward_tiled<0, 0, 0, 0>), grid, block, bytes, st, derInput, x, derOutput, p, t, (int)strips);
      return check_launch("mcn_pool_backward_f64");
    }
  }
  KernelTimer timer("pool64_backward", as_stream(stream));
  if (isMax)
    hipLaunchKernelGGL(pool64_backward<true>, dim3(blocks), dim3(256), 0, as_stream(stream), derInput, x, derOutput, p, total);
  else
    hipLaunchKernelGGL(pool64_backward<false>, dim3(blocks), dim3(256), 0, as_stream(stream), derInput, x, derOutput, p, total);
  return check_launch("mcn_pool_backward_f64");
}

}  // extern "C"
