// Pooling forward / backward for gfx950.
//
// Backward is a GATHER: one accumulator per input element, no atomics.  For every input element the
// outputs whose window covers it are visited in the order the reference CPU loop visits them (output
// column ascending, then output row ascending; bits/nnpooling.cu:190-206), starting from +0.0f (or from
// the existing value when accumulating), and every addition is a separate IEEE add.  That reproduces
// the reference's float sums bit for bit, which the CUDA reference (atomicAdd per output,
// bits/nnpooling_gpu.cu:158-165) does not guarantee.
//
// Max pooling: the winner of a window is the first element, scanning the clipped window column by
// column, that is strictly greater than all before it, starting from -inf (acc_max,
// bits/nnpooling.cu:33-66).  NaN never wins; an all-NaN / all -inf window routes nothing.
//
// Tiled kernel: a workgroup owns all H rows of TW input columns of one (channel,image) plane.  It stages
// in LDS the x columns touched by the windows of every output that covers the tile (contiguous in
// memory), the matching dzdy columns, computes each such output's winner once, then gathers.  HBM sees
// x once (+ halo columns), dzdy once (+ halo), dzdx once.
#include "mcn_internal.hpp"

#include <algorithm>

// Every multiply and add below must stay a separate IEEE operation: results are compared bit for bit
// with the reference CPU loops, so fused multiply-add contraction is switched off for this file.
#pragma clang fp contract(off)

namespace mcn {
namespace {

struct PoolP {
  int H, W, outH, outW;
  int poolH, poolW, sy, sx, pt, pl;
  int TW, tilesPerPlane;
  int accumulate;
};

__device__ __forceinline__ int ceil_div_clamp0(int a, int b) { return a <= 0 ? 0 : (a + b - 1) / b; }

// 1 / (clipped window area) of output (oh, ow), computed like acc_sum: T(1)/T(h*w) (bits/nnpooling.cu:74)
__device__ __forceinline__ float avg_scale(const PoolP& p, int oh, int ow) {
  int h1 = oh * p.sy - p.pt, w1 = ow * p.sx - p.pl;
  int h2 = min(h1 + p.poolH, p.H), w2 = min(w1 + p.poolW, p.W);
  h1 = max(h1, 0);
  w1 = max(w1, 0);
  return 1.0f / (float)((h2 - h1) * (w2 - w1));  // correctly rounded IEEE division
}

template <bool MAX, bool VEC4>
__global__ __launch_bounds__(256) void pool_backward_tiled(float* __restrict__ dx,
                                                           const float* __restrict__ x,
                                                           const float* __restrict__ dy, PoolP p) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int z = logical / p.tilesPerPlane;
  const int tile = logical - z * p.tilesPerPlane;
  const int w0 = tile * p.TW;
  const int w1 = min(w0 + p.TW, p.W);

  // outputs whose window touches columns [w0, w1)
  const int owLo = ceil_div_clamp0(w0 + p.pl - p.poolW + 1, p.sx);
  const int owHi = min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);  // inclusive
  const int nOW = max(owHi - owLo + 1, 0);
  const int nOut = nOW * p.outH;
  // x columns read by those windows
  const int wa = max(owLo * p.sx - p.pl, 0);
  const int wb = (nOW > 0) ? min(owHi * p.sx - p.pl + p.poolW, p.W) : wa;
  const int nX = MAX ? (wb - wa) * p.H : 0;

  float* xs = smem;                 // [nX]   (max only)
  float* dys = smem + nX;           // [nOut]
  int* win = (int*)(dys + nOut);    // [nOut] (max only)

  const size_t planeIn = (size_t)z * p.H * p.W;
  const size_t planeOut = (size_t)z * p.outH * p.outW;

  // ---- stage x columns and dzdy columns (both contiguous ranges of their planes)
  if (MAX) {
    const float* src = x + planeIn + (size_t)wa * p.H;
    if (VEC4) {
      const float4* s4 = (const float4*)src;
      float4* d4 = (float4*)xs;
      for (int i = tid; i < nX / 4; i += 256) d4[i] = s4[i];
    } else {
      for (int i = tid; i < nX; i += 256) xs[i] = src[i];
    }
  }
  {
    const float* src = dy + planeOut + (size_t)owLo * p.outH;
    if (VEC4) {
      const float4* s4 = (const float4*)src;
      float4* d4 = (float4*)dys;
      for (int i = tid; i < nOut / 4; i += 256) d4[i] = s4[i];
    } else {
      for (int i = tid; i < nOut; i += 256) dys[i] = src[i];
    }
  }
  __syncthreads();

  // ---- winner of every staged output (linear index inside the plane, -1 = none)
  if (MAX) {
    for (int o = tid; o < nOut; o += 256) {
      const int owr = o / p.outH;
      const int oh = o - owr * p.outH;
      const int ow = owLo + owr;
      int h1 = oh * p.sy - p.pt, c1 = ow * p.sx - p.pl;
      const int h2 = min(h1 + p.poolH, p.H), c2 = min(c1 + p.poolW, p.W);
      h1 = max(h1, 0);
      c1 = max(c1, 0);
      float best = -INFINITY;
      int bi = -1;
      for (int w = c1; w < c2; ++w) {
        const float* col = xs + (w - wa) * p.H;
        for (int h = h1; h < h2; ++h) {
          const float v = col[h];
          if (v > best) {
            best = v;
            bi = w * p.H + h;
          }
        }
      }
      win[o] = bi;
    }
    __syncthreads();
  }

  // ---- gather: one accumulator per input element of the tile
  auto gather = [&](int h, int w, float acc) -> float {
    const int ohA = ceil_div_clamp0(h + p.pt - p.poolH + 1, p.sy);
    const int ohB = min(p.outH - 1, (h + p.pt) / p.sy);
    const int owA = ceil_div_clamp0(w + p.pl - p.poolW + 1, p.sx);
    const int owB = min(p.outW - 1, (w + p.pl) / p.sx);
    const int me = w * p.H + h;
    for (int ow = owA; ow <= owB; ++ow) {
      const int base = (ow - owLo) * p.outH;
      for (int oh = ohA; oh <= ohB; ++oh) {
        if (MAX) {
          if (win[base + oh] == me) acc = acc + dys[base + oh];
        } else {
          {
            const float term = dys[base + oh] * avg_scale(p, oh, ow);  // rounded product, then a separate add
            acc = acc + term;
          }
        }
      }
    }
    return acc;
  };

  float* out = dx + planeIn + (size_t)w0 * p.H;
  const int nIn = (w1 - w0) * p.H;
  if (VEC4) {
    float4* o4 = (float4*)out;
    for (int e = tid; e < nIn / 4; e += 256) {
      const int lin = e * 4;
      const int wr = lin / p.H;
      const int h = lin - wr * p.H;
      const int w = w0 + wr;
      float4 a = p.accumulate ? o4[e] : make_float4(0.f, 0.f, 0.f, 0.f);
      a.x = gather(h, w, a.x);
      a.y = gather(h + 1, w, a.y);
      a.z = gather(h + 2, w, a.z);
      a.w = gather(h + 3, w, a.w);
      o4[e] = a;
    }
  } else {
    for (int e = tid; e < nIn; e += 256) {
      const int wr = e / p.H;
      const int h = e - wr * p.H;
      const float a = p.accumulate ? out[e] : 0.f;
      out[e] = gather(h, w0 + wr, a);
    }
  }
}

// Fallback without LDS staging (planes too tall for a tile): one thread per input element, winners
// recomputed from global memory.  Same visiting order, same results.
template <bool MAX>
__global__ __launch_bounds__(256) void pool_backward_direct(float* __restrict__ dx,
                                                            const float* __restrict__ x,
                                                            const float* __restrict__ dy, PoolP p,
                                                            size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int plane = p.H * p.W;
  const size_t z = idx / plane;
  const int me = (int)(idx - z * plane);
  const int w = me / p.H;
  const int h = me - w * p.H;
  const float* xp = x + z * plane;
  const float* dyp = dy + z * (size_t)p.outH * p.outW;
  const int ohA = ceil_div_clamp0(h + p.pt - p.poolH + 1, p.sy);
  const int ohB = min(p.outH - 1, (h + p.pt) / p.sy);
  const int owA = ceil_div_clamp0(w + p.pl - p.poolW + 1, p.sx);
  const int owB = min(p.outW - 1, (w + p.pl) / p.sx);
  float acc = p.accumulate ? dx[idx] : 0.f;
  for (int ow = owA; ow <= owB; ++ow)
    for (int oh = ohA; oh <= ohB; ++oh) {
      const float d = dyp[ow * p.outH + oh];
      if (MAX) {
        int h1 = oh * p.sy - p.pt, c1 = ow * p.sx - p.pl;
        const int h2 = min(h1 + p.poolH, p.H), c2 = min(c1 + p.poolW, p.W);
        h1 = max(h1, 0);
        c1 = max(c1, 0);
        float best = -INFINITY;
        int bi = -1;
        for (int ww = c1; ww < c2; ++ww)
          for (int hh = h1; hh < h2; ++hh) {
            const float v = xp[ww * p.H + hh];
            if (v > best) {
              best = v;
              bi = ww * p.H + hh;
            }
          }
        if (bi == me) acc = acc + d;
      } else {
        {
        const float term = d * avg_scale(p, oh, ow);
        acc = acc + term;
      }
      }
    }
  dx[idx] = acc;
}

// Forward: one thread per output element (PoolingForwardCPU, bits/nnpooling.cu:102-142).
template <bool MAX>
__global__ __launch_bounds__(256) void pool_forward_kernel(float* __restrict__ y,
                                                           const float* __restrict__ x, PoolP p,
                                                           size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int oplane = p.outH * p.outW;
  const size_t z = idx / oplane;
  const int o = (int)(idx - z * oplane);
  const int ow = o / p.outH;
  const int oh = o - ow * p.outH;
  const float* xp = x + z * (size_t)p.H * p.W;
  int h1 = oh * p.sy - p.pt, c1 = ow * p.sx - p.pl;
  const int h2 = min(h1 + p.poolH, p.H), c2 = min(c1 + p.poolW, p.W);
  h1 = max(h1, 0);
  c1 = max(c1, 0);
  if (MAX) {
    float best = -INFINITY;
    for (int w = c1; w < c2; ++w)
      for (int h = h1; h < h2; ++h) {
        const float v = xp[w * p.H + h];
        best = (best < v) ? v : best;  // std::max(best, v): NaN never replaces best
      }
    y[idx] = best;
  } else {
    float s = 0.f;
    for (int w = c1; w < c2; ++w)
      for (int h = h1; h < h2; ++h) s = s + xp[w * p.H + h];
    y[idx] = s * (1.0f / (float)((h2 - h1) * (c2 - c1)));
  }
}

int validate(const mcn_pool_geom* g, const char* who, PoolP* p) {
  if (!g) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null geometry", who);
  if (g->H < 0 || g->W < 0 || g->C < 0 || g->N < 0)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if (g->poolH < 1 || g->poolW < 1) return fail(MCN_ILLEGAL_ARGUMENT, "%s: a dimension of POOL is void", who);
  if (g->strideY < 1 || g->strideX < 1)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: at least one element of STRIDE is smaller than one", who);
  if (g->padTop < 0 || g->padBottom < 0 || g->padLeft < 0 || g->padRight < 0)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: an element of PAD is negative", who);
  if (g->H + g->padTop + g->padBottom < g->poolH || g->W + g->padLeft + g->padRight < g->poolW)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: the pooling window is larger than the DATA (including padding)", who);
  if (g->method != MCN_POOL_MAX && g->method != MCN_POOL_AVERAGE)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: unknown pooling method %d", who, g->method);
  if ((long long)g->H * g->W >= (1ll << 31))
    return fail(MCN_UNSUPPORTED, "%s: a plane of more than 2^31 elements is not supported", who);
  p->H = g->H;
  p->W = g->W;
  p->outH = (g->H + g->padTop + g->padBottom - g->poolH) / g->strideY + 1;
  p->outW = (g->W + g->padLeft + g->padRight - g->poolW) / g->strideX + 1;
  p->poolH = g->poolH;
  p->poolW = g->poolW;
  p->sy = g->strideY;
  p->sx = g->strideX;
  p->pt = g->padTop;
  p->pl = g->padLeft;
  p->TW = 0;
  p->tilesPerPlane = 0;
  p->accumulate = 0;
  return MCN_SUCCESS;
}

// LDS bytes the tiled kernel needs for tile width TW (maximum over the tiles of a plane).
size_t tile_lds_bytes(const PoolP& p, bool isMax, int TW) {
  size_t worst = 0;
  for (int w0 = 0; w0 < p.W; w0 += TW) {
    const int w1 = std::min(w0 + TW, p.W);
    const int num = w0 + p.pl - p.poolW + 1;
    const int owLo = num <= 0 ? 0 : (num + p.sx - 1) / p.sx;
    const int owHi = std::min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);
    const int nOW = std::max(owHi - owLo + 1, 0);
    const int wa = std::max(owLo * p.sx - p.pl, 0);
    const int wb = nOW > 0 ? std::min(owHi * p.sx - p.pl + p.poolW, p.W) : wa;
    size_t need = (size_t)nOW * p.outH * sizeof(float);
    if (isMax) need += (size_t)(wb - wa) * p.H * sizeof(float) + (size_t)nOW * p.outH * sizeof(int);
    worst = std::max(worst, need);
  }
  return worst;
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

int mcn_pool_output_size(const mcn_pool_geom* g, int* outH, int* outW) {
  PoolP p;
  int rc = validate(g, "mcn_pool_output_size", &p);
  if (rc) return rc;
  if (outH) *outH = p.outH;
  if (outW) *outW = p.outW;
  return MCN_SUCCESS;
}

int mcn_pool_forward(mcn_stream_t stream, const mcn_pool_geom* g, float* y, const float* x) {
  PoolP p;
  int rc = validate(g, "mcn_pool_forward", &p);
  if (rc) return rc;
  const size_t total = (size_t)p.outH * p.outW * g->C * g->N;
  if (total == 0) return MCN_SUCCESS;
  if (!y || !x) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_pool_forward: null tensor");
  const size_t blocks = (total + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "mcn_pool_forward: tensor too large");
  if (g->method == MCN_POOL_MAX)
    hipLaunchKernelGGL(pool_forward_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), y, x, p, total);
  else
    hipLaunchKernelGGL(pool_forward_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), y, x, p, total);
  return check_launch("mcn_pool_forward");
}

int mcn_pool_backward(mcn_stream_t stream, const mcn_pool_geom* g, float* derInput, const float* x,
                      const float* derOutput, int accumulate) {
  PoolP p;
  int rc = validate(g, "mcn_pool_backward", &p);
  if (rc) return rc;
  const size_t planes = (size_t)g->C * g->N;
  const size_t total = planes * p.H * p.W;
  if (total == 0) return MCN_SUCCESS;
  const bool isMax = g->method == MCN_POOL_MAX;
  if (!derInput || !derOutput || (isMax && !x)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_pool_backward: null tensor");
  p.accumulate = accumulate ? 1 : 0;
  hipStream_t s = as_stream(stream);

  // widest tile (fewest tiles per plane) whose staging fits the LDS budget
  const size_t budget = (size_t)std::min(std::max(tunable("pool_lds_bytes", 24 * 1024), 1024), 64 * 1024);
  int tiles = 0;
  size_t lds = 0;
  for (int nT = 1; nT <= p.W; ++nT) {
    const int TW = (p.W + nT - 1) / nT;
    if (nT > 1 && TW == (p.W + nT - 2) / (nT - 1)) continue;  // same width as the previous candidate
    const size_t need = tile_lds_bytes(p, isMax, TW);
    if (need <= budget) {
      tiles = (p.W + TW - 1) / TW;
      p.TW = TW;
      lds = need;
      break;
    }
  }
  if (tiles > 0 && planes * tiles < (1ull << 31)) {
    p.tilesPerPlane = tiles;
    const bool vec = (p.H % 4 == 0) && (p.outH % 4 == 0) && aligned16(derInput) && aligned16(derOutput) &&
                     (!isMax || aligned16(x));
    const dim3 grid((unsigned)(planes * tiles)), block(256);
    KernelTimer timer("pool_backward_tiled", s);
    if (isMax) {
      if (vec) hipLaunchKernelGGL((pool_backward_tiled<true, true>), grid, block, lds, s, derInput, x, derOutput, p);
      else hipLaunchKernelGGL((pool_backward_tiled<true, false>), grid, block, lds, s, derInput, x, derOutput, p);
    } else {
      if (vec) hipLaunchKernelGGL((pool_backward_tiled<false, true>), grid, block, lds, s, derInput, x, derOutput, p);
      else hipLaunchKernelGGL((pool_backward_tiled<false, false>), grid, block, lds, s, derInput, x, derOutput, p);
    }
    return check_launch("mcn_pool_backward");
  }
  const size_t blocks = (total + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "mcn_pool_backward: tensor too large");
  if (isMax)
    hipLaunchKernelGGL(pool_backward_direct<true>, dim3((unsigned)blocks), dim3(256), 0, s, derInput, x, derOutput, p, total);
  else
    hipLaunchKernelGGL(pool_backward_direct<false>, dim3((unsigned)blocks), dim3(256), 0, s, derInput, x, derOutput, p, total);
  return check_launch("mcn_pool_backward");
}

}  // extern "C"
