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

bool pool_max_backward_pairs_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, float* derInput,
                                    const float* x, const float* derOutput, int accumulate);  // pool_pairs.hip
bool pool_max_backward_stream_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, float* derInput,
                                     const float* x, const float* derOutput, int accumulate);  // pool_stream.hip

namespace {

struct PoolP {
  int H, W, outH, outW;
  int poolH, poolW, sy, sx, pt, pl;
  int TW, tilesPerPlane;
  int accumulate;
  // rank of an output among the outputs covering its winner: min(o, rankTab[window offset of the winner]),
  // rankTab[i] = (pool - 1 - i) / stride   (windows up to 8 x 8)
  int rankH[8], rankW[8];
  // host-precomputed helpers of the ordered-pass kernel (no integer division on the device)
  FastDiv byTiles, bySx, byOutH, byStageRow, byBorder;  // stage row = H/4 (16-byte staging) or H; border rows per column
  int outStepQ, outStepR;      // 256 = outStepQ * outH + outStepR
  int stageStepQ, stageStepR;  // 256 = stageStepQ * stageRow + stageStepR
  int KH, nPasses;
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

// Copies n floats global -> LDS with four independent 16-byte (or 4-byte) loads in flight per thread.
template <bool VEC4>
__device__ __forceinline__ void stage(float* __restrict__ dst, const float* __restrict__ src, int n, int tid) {
  if (VEC4) {
    const int n4 = n / 4;
    for (int base = 0; base < n4; base += 4 * 256) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * 256 + tid;
        if (i < n4) v[u] = ((const float4*)src)[i];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * 256 + tid;
        if (i < n4) ((float4*)dst)[i] = v[u];
      }
    }
  } else {
    for (int base = 0; base < n; base += 4 * 256) {
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * 256 + tid;
        if (i < n) v[u] = src[i];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * 256 + tid;
        if (i < n) dst[i] = v[u];
      }
    }
  }
}

// Covering outputs of input row h (resp. column w): o with o*stride - pad <= h < o*stride - pad + pool,
// clipped to [0, nOut).  Packed as lo | hi << 16 (hi inclusive; lo > hi when nothing covers).
__device__ __forceinline__ int cover_range(int h, int pad, int pool, int stride, int nOut) {
  const int lo = ceil_div_clamp0(h + pad - pool + 1, stride);
  const int hi = min(nOut - 1, (h + pad) / stride);
  return (lo & 0xffff) | (hi << 16);
}

// Average pooling whose single window covers the whole plane: dx = [dx +] dy[plane] * (1 / (H*W)).
__global__ __launch_bounds__(256) void pool_avg_backward_whole(float* __restrict__ dx, const float* __restrict__ dy,
                                                               unsigned total, unsigned planeSize, int accumulate) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const float scale = 1.0f / (float)planeSize;  // as avg_scale: correctly rounded IEEE division
  const float v = dy[i / planeSize] * scale;
  dx[i] = (accumulate ? dx[i] : 0.0f) + v;  // (0 + v, as the general kernels' sum starts: -0 becomes +0)
}

// Average pooling whose windows tile the plane exactly (pool = stride, no padding, H = outH * poolH, W = outW *
// poolW; H a multiple of 4): every input element lies in exactly one whole window, dx = [dx +] dy[its window] * (1 /
// (poolH * poolW)).  One thread per 16 bytes of dx, in memory order: a plain streaming kernel (reads dzdy once -- the
// poolH * poolW threads that share a window hit L1 -- and writes dx once).
// E: float or double; a thread's 16 bytes are VE = 4 or 2 elements (H4 = H / VE cells per column).
template <typename E>
__global__ __launch_bounds__(256) void pool_backward_avg_tiles(E* __restrict__ dx, const E* __restrict__ dy, unsigned total4,
                                                               int H4, int W, int outH, int outW, FastDiv byH4, FastDiv byW,
                                                               FastDiv byPh, FastDiv byPw, int poolArea, int accumulate) {
  constexpr int VE = 16 / sizeof(E);
  typedef E vec __attribute__((ext_vector_type(VE)));
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total4) return;
  int col, q, plane, w;
  byH4.divmod((int)i, &col, &q);     // i = (plane * W + w) * H4 + q
  byW.divmod(col, &plane, &w);
  const E scale = (E)1 / (E)poolArea;  // as avg_scale: correctly rounded IEEE division
  const E* src = dy + ((size_t)plane * outW + byPw.div(w)) * outH;
  E v[VE];
#pragma unroll
  for (int r = 0; r < VE; ++r) v[r] = src[byPh.div(VE * q + r)] * scale;
  vec out = (vec)(E)0;  // (0 + v, as the general kernels' sum starts: -0 becomes +0)
  if (accumulate) out = ((const vec*)dx)[i];
#pragma unroll
  for (int r = 0; r < VE; ++r) out[r] = out[r] + v[r];
#if MCN_NT_STORE
  __builtin_nontemporal_store(out, (vec*)dx + i);
#else
  ((vec*)dx)[i] = out;
#endif
}

// Launches it when the windows tile the plane exactly and its columns are whole 16-byte cells; false otherwise.
template <typename E>
bool avg_tiles_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, E* derInput, const E* derOutput,
                      int accumulate) {
  constexpr int VE = 16 / sizeof(E);
  const size_t total = (size_t)g->C * g->N * g->H * g->W;
  if (g->method == MCN_POOL_MAX || g->poolH != g->strideY || g->poolW != g->strideX || g->padTop != 0 || g->padLeft != 0 ||
      g->H != outH * g->poolH || g->W != outW * g->poolW || g->H % VE != 0 || !aligned16(derInput) ||
      total / VE >= (1ull << 31) || tunable("pool_force_gather", 0))
    return false;
  KernelTimer timer("pool_backward_avg_tiles", s);
  hipLaunchKernelGGL(pool_backward_avg_tiles<E>, dim3((unsigned)((total / VE + 255) / 256)), dim3(256), 0, s, derInput,
                     derOutput, (unsigned)(total / VE), g->H / VE, g->W, outH, outW, FastDiv(g->H / VE), FastDiv(g->W),
                     FastDiv(g->poolH), FastDiv(g->poolW), g->poolH * g->poolW, accumulate ? 1 : 0);
  return true;
}

// KH, KW: upper bounds on the number of output rows / columns covering one input element
// (ceil(pool/stride)); 0 selects run-time loops.  With compile-time bounds the candidate loads are issued
// together and the adds are predicated, which keeps the reference's addition order.
template <bool MAX, bool VEC4, int KH, int KW>
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
  const int Hpad = (p.H + 3) & ~3;

  // LDS carve-up (every piece a multiple of 4 floats so 16-byte accesses stay aligned)
  int* rowCover = (int*)smem;                  // [Hpad]  covering output rows of each input row
  int* colCover = rowCover + Hpad;             // [TWpad] covering output columns of each tile column
  float* xs = (float*)(colCover + ((p.TW + 3) & ~3));  // [nX]   staged x columns        (max only)
  float* dys = xs + ((nX + 3) & ~3);           // [nOut] staged dzdy (avg: already multiplied by 1/area)
  int* win = (int*)(dys + ((nOut + 3) & ~3));  // [nOut] winner of each staged output    (max only)

  const size_t planeIn = (size_t)z * p.H * p.W;
  const size_t planeOut = (size_t)z * p.outH * p.outW;

  // ---- stage x columns and dzdy columns (both contiguous ranges of their planes); cover tables
  stage<VEC4>(dys, dy + planeOut + (size_t)owLo * p.outH, nOut, tid);
  if (MAX) stage<VEC4>(xs, x + planeIn + (size_t)wa * p.H, nX, tid);
  for (int h = tid; h < p.H; h += 256) rowCover[h] = cover_range(h, p.pt, p.poolH, p.sy, p.outH);
  for (int c = tid; c < w1 - w0; c += 256) colCover[c] = cover_range(w0 + c, p.pl, p.poolW, p.sx, p.outW);
  __syncthreads();

  // ---- per staged output: its winner (max) or its share dzdy/area (avg).  (owr, oh) advance without divisions.
  {
    int owr = tid / p.outH, oh = tid - owr * p.outH;
    const int stepQ = 256 / p.outH, stepR = 256 - stepQ * p.outH;
    for (int o = tid; o < nOut; o += 256) {
      const int ow = owLo + owr;
      int h1 = oh * p.sy - p.pt, c1 = ow * p.sx - p.pl;
      const int h2 = min(h1 + p.poolH, p.H), c2 = min(c1 + p.poolW, p.W);
      h1 = max(h1, 0);
      c1 = max(c1, 0);
      if (MAX) {
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
      } else {
        // derOutput * scale with scale = T(1)/T(clipped area), rounded like acc_sum (bits/nnpooling.cu:68-96)
        dys[o] = dys[o] * (1.0f / (float)((h2 - h1) * (c2 - c1)));
      }
      owr += stepQ;
      oh += stepR;
      if (oh >= p.outH) {
        oh -= p.outH;
        ++owr;
      }
    }
  }
  __syncthreads();

  // ---- gather: one accumulator per input element of the tile; covering outputs visited column-major
  auto gather = [&](int me, int rc, int cc, float acc) -> float {
    const int ohA = rc & 0xffff, ohB = rc >> 16;
    const int owA = cc & 0xffff, owB = cc >> 16;
    if (KH > 0 && KW > 0) {
      float d[KW > 0 ? KW : 1][KH > 0 ? KH : 1];
      bool hit[KW > 0 ? KW : 1][KH > 0 ? KH : 1];
#pragma unroll
      for (int b = 0; b < KW; ++b) {
        const int ow = owA + b;
        const int base = (ow - owLo) * p.outH;
#pragma unroll
        for (int a = 0; a < KH; ++a) {
          const int oh = ohA + a;
          const bool ok = ow <= owB && oh <= ohB;
          const int idx = ok ? base + oh : 0;
          d[b][a] = dys[idx];
          hit[b][a] = ok && (!MAX || win[idx] == me);
        }
      }
#pragma unroll
      for (int b = 0; b < KW; ++b)
#pragma unroll
        for (int a = 0; a < KH; ++a)
          if (hit[b][a]) acc = acc + d[b][a];
      return acc;
    }
    for (int ow = owA; ow <= owB; ++ow) {
      const int base = (ow - owLo) * p.outH;
      for (int oh = ohA; oh <= ohB; ++oh) {
        if (MAX) {
          if (win[base + oh] == me) acc = acc + dys[base + oh];
        } else {
          acc = acc + dys[base + oh];
        }
      }
    }
    return acc;
  };

  float* out = dx + planeIn + (size_t)w0 * p.H;
  const int nIn = (w1 - w0) * p.H;
  if (VEC4) {
    float4* o4 = (float4*)out;
    const int HQ = p.H / 4;
    int wr = tid / HQ, hq = tid - wr * HQ;
    const int stepQ = 256 / HQ, stepR = 256 - stepQ * HQ;
    for (int e = tid; e < nIn / 4; e += 256) {
      const int h = hq * 4;
      const int4 rc = *(const int4*)(rowCover + h);
      const int cc = colCover[wr];
      const int me = (w0 + wr) * p.H + h;
      float4 a = p.accumulate ? o4[e] : make_float4(0.f, 0.f, 0.f, 0.f);
      a.x = gather(me, rc.x, cc, a.x);
      a.y = gather(me + 1, rc.y, cc, a.y);
      a.z = gather(me + 2, rc.z, cc, a.z);
      a.w = gather(me + 3, rc.w, cc, a.w);
      o4[e] = a;
      wr += stepQ;
      hq += stepR;
      if (hq >= HQ) {
        hq -= HQ;
        ++wr;
      }
    }
  } else {
    int wr = tid / p.H, h = tid - wr * p.H;
    const int stepQ = 256 / p.H, stepR = 256 - stepQ * p.H;
    for (int e = tid; e < nIn; e += 256) {
      const float a = p.accumulate ? out[e] : 0.f;
      out[e] = gather((w0 + wr) * p.H + h, rowCover[h], colCover[wr], a);
      wr += stepQ;
      h += stepR;
      if (h >= p.H) {
        h -= p.H;
        ++wr;
      }
    }
  }
}

// Max pooling, compile-time cover bounds KH x KW (<= 32 combinations).  Same tiling as above, but instead of
// every input element asking each covering output "did I win?", every output tells its winner: after
// computing its winner it sets bit (b*KH + a) in that element's flag word (LDS atomic OR, order
// independent), where (a, b) is the output's position among the outputs covering the winner.  Three
// quarters of the input elements of a 3x3/stride-2 pooling win nothing and are finished after one flag
// read; winners add their dzdy values in ascending bit order, which is the reference's visiting order
// (output column, then output row).
// PH, PW: compile-time pooling window (0 = run-time loops): the window's loads are then issued together and
// elements outside the clipped window are skipped by predicate, in the same scan order.
template <bool VEC4, int KH, int KW, int PH, int PW>
__global__ __launch_bounds__(256) void pool_max_backward_flags(float* __restrict__ dx,
                                                               const float* __restrict__ x,
                                                               const float* __restrict__ dy, PoolP p) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int z = logical / p.tilesPerPlane;
  const int tile = logical - z * p.tilesPerPlane;
  const int w0 = tile * p.TW;
  const int w1 = min(w0 + p.TW, p.W);
  const int owLo = ceil_div_clamp0(w0 + p.pl - p.poolW + 1, p.sx);
  const int owHi = min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);
  const int nOW = max(owHi - owLo + 1, 0);
  const int nOut = nOW * p.outH;
  const int wa = max(owLo * p.sx - p.pl, 0);
  const int wb = (nOW > 0) ? min(owHi * p.sx - p.pl + p.poolW, p.W) : wa;
  const int nX = (wb - wa) * p.H;
  const int nIn = (w1 - w0) * p.H;
  const int Hpad = (p.H + 3) & ~3;

  int* rowCover = (int*)smem;                              // [Hpad]
  int* colCover = rowCover + Hpad;                         // [TWpad]
  float* xs = (float*)(colCover + ((p.TW + 3) & ~3));      // [nX]
  float* dys = xs + ((nX + 3) & ~3);                       // [nOut]
  unsigned* flags = (unsigned*)(dys + ((nOut + 3) & ~3));  // [TW*H]

  const size_t planeIn = (size_t)z * p.H * p.W;
  const size_t planeOut = (size_t)z * p.outH * p.outW;
  stage<VEC4>(xs, x + planeIn + (size_t)wa * p.H, nX, tid);
  stage<VEC4>(dys, dy + planeOut + (size_t)owLo * p.outH, nOut, tid);
  if (VEC4) {
    for (int i = tid; i < nIn / 4; i += 256) ((uint4*)flags)[i] = make_uint4(0u, 0u, 0u, 0u);
  } else {
    for (int i = tid; i < nIn; i += 256) flags[i] = 0u;
  }
  for (int h = tid; h < p.H; h += 256) rowCover[h] = cover_range(h, p.pt, p.poolH, p.sy, p.outH);
  for (int c = tid; c < w1 - w0; c += 256) colCover[c] = cover_range(w0 + c, p.pl, p.poolW, p.sx, p.outW);
  __syncthreads();

  // ---- every staged output finds its winner and flags it
  {
    int owr = tid / p.outH, oh = tid - owr * p.outH;
    const int stepQ = 256 / p.outH, stepR = 256 - stepQ * p.outH;
    for (int o = tid; o < nOut; o += 256) {
      const int ow = owLo + owr;
      int h1 = oh * p.sy - p.pt, c1 = ow * p.sx - p.pl;
      const int h2 = min(h1 + p.poolH, p.H), c2 = min(c1 + p.poolW, p.W);
      h1 = max(h1, 0);
      c1 = max(c1, 0);
      float best = -INFINITY;
      int bh = -1, bw = 0;
      if (PH > 0 && PW > 0) {
        const int hu = oh * p.sy - p.pt, cu = ow * p.sx - p.pl;  // unclipped window origin
        float v[PW > 0 ? PW : 1][PH > 0 ? PH : 1];
#pragma unroll
        for (int j = 0; j < PW; ++j)
#pragma unroll
          for (int i = 0; i < PH; ++i) {
            const int h = hu + i, w = cu + j;
            const bool in = h >= h1 && h < h2 && w >= c1 && w < c2;
            v[j][i] = in ? xs[(w - wa) * p.H + h] : -INFINITY;  // -inf never beats the start value
          }
#pragma unroll
        for (int j = 0; j < PW; ++j)
#pragma unroll
          for (int i = 0; i < PH; ++i)
            if (v[j][i] > best) {
              best = v[j][i];
              bh = hu + i;
              bw = cu + j;
            }
      } else {
        for (int w = c1; w < c2; ++w) {
          const float* col = xs + (w - wa) * p.H;
          for (int h = h1; h < h2; ++h) {
            const float v = col[h];
            if (v > best) {
              best = v;
              bh = h;
              bw = w;
            }
          }
        }
      }
      if (bh >= 0 && bw >= w0 && bw < w1) {
        const int a = oh - (rowCover[bh] & 0xffff);
        const int b = ow - (colCover[bw - w0] & 0xffff);
        atomicOr(&flags[(bw - w0) * p.H + bh], 1u << (b * KH + a));
      }
      owr += stepQ;
      oh += stepR;
      if (oh >= p.outH) {
        oh -= p.outH;
        ++owr;
      }
    }
  }
  __syncthreads();

  // ---- winners collect their dzdy in ascending bit order
  auto collect = [&](unsigned f, int h, int wr, float acc) -> float {
    if (f == 0u) return acc;
    const int ohA = rowCover[h] & 0xffff;
    const int owA = colCover[wr] & 0xffff;
    while (f) {
      const int t = __ffs(f) - 1;
      f &= f - 1u;
      const int b = t / KH, a = t - b * KH;
      acc = acc + dys[(owA + b - owLo) * p.outH + ohA + a];
    }
    return acc;
  };

  float* out = dx + planeIn + (size_t)w0 * p.H;
  if (VEC4) {
    float4* o4 = (float4*)out;
    const int HQ = p.H / 4;
    int wr = tid / HQ, hq = tid - wr * HQ;
    const int stepQ = 256 / HQ, stepR = 256 - stepQ * HQ;
    for (int e = tid; e < nIn / 4; e += 256) {
      const uint4 f = ((const uint4*)flags)[e];
      float4 a = p.accumulate ? o4[e] : make_float4(0.f, 0.f, 0.f, 0.f);
      if (f.x | f.y | f.z | f.w) {
        const int h = hq * 4;
        a.x = collect(f.x, h, wr, a.x);
        a.y = collect(f.y, h + 1, wr, a.y);
        a.z = collect(f.z, h + 2, wr, a.z);
        a.w = collect(f.w, h + 3, wr, a.w);
      }
      o4[e] = a;
      wr += stepQ;
      hq += stepR;
      if (hq >= HQ) {
        hq -= HQ;
        ++wr;
      }
    }
  } else {
    int wr = tid / p.H, h = tid - wr * p.H;
    const int stepQ = 256 / p.H, stepR = 256 - stepQ * p.H;
    for (int e = tid; e < nIn; e += 256) {
      const float a = p.accumulate ? out[e] : 0.f;
      out[e] = collect(flags[e], h, wr, a);
      wr += stepQ;
      h += stepR;
      if (h >= p.H) {
        h -= p.H;
        ++wr;
      }
    }
  }
}

// Ordered-pass kernel (the fast path).  A workgroup owns all rows of TW columns of one plane and keeps one fp32
// accumulator per owned input element in LDS, initialised to +0 (or to derInput when accumulating).  Each
// thread owns up to OPT of the outputs whose windows touch the tile, with their dzdy in registers.
//   max: the x columns those windows read are staged in LDS inside a -inf frame (so windows need no
//        clipping tests); each output finds its winner once and its rank t among the outputs covering that
//        winner (t = column rank * KH + row rank).  Then KH*KW barrier-separated passes: in pass t the
//        outputs of rank t add their dzdy to their winner's accumulator.  Within a pass an accumulator is
//        touched by at most one output, and across passes an input's contributions arrive in ascending
//        (output column, output row) order -- the order of the reference loop (bits/nnpooling.cu:190-206).
//   avg: PH*PW passes over window positions in descending (column, row) order; in a pass every output adds
//        dzdy * (1/clipped area) to the one element at that window position, which again visits each input's
//        outputs in ascending (output column, output row) order.
// The final accumulators are streamed out with 16-byte stores.  No atomics, results bit-identical to the CPU.
template <bool MAX, bool VEC4, int OPT, int PH, int PW>
__global__ __launch_bounds__(256) void pool_backward_passes(float* __restrict__ dx,
                                                            const float* __restrict__ x,
                                                            const float* __restrict__ dy, PoolP p) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x;
  const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
  int z, tile;
  p.byTiles.divmod(logical, &z, &tile);
  const int w0 = tile * p.TW;
  const int w1 = min(w0 + p.TW, p.W);
  const int loNum = w0 + p.pl - p.poolW + 1;
  const int owLo = loNum <= 0 ? 0 : p.bySx.div(loNum + p.sx - 1);
  const int owHi = min(p.outW - 1, p.bySx.div(w1 - 1 + p.pl));
  const int nOW = max(owHi - owLo + 1, 0);
  const int nOut = nOW * p.outH;
  const int nIn = (w1 - w0) * p.H;
  const int poolH = PH > 0 ? PH : p.poolH, poolW = PW > 0 ? PW : p.poolW;
  // framed staging area: frame column c <-> image column cLo + c, frame row r <-> image row r - pt
  const int cLo = owLo * p.sx - p.pl;
  const int nC = MAX && nOW > 0 ? (owHi - owLo) * p.sx + poolW : 0;
  // frame pitch: every row a window can read, and never less than the rows the interior copy writes
  const int Hp = max((p.outH - 1) * p.sy + poolH, p.pt + p.H);

  float* acc = smem;                    // [nIn] one accumulator per owned input element
  float* xs = acc + ((nIn + 3) & ~3);   // [nC*Hp] x inside a -inf frame (max only)

  const size_t planeIn = (size_t)z * p.H * p.W;
  const size_t planeOut = (size_t)z * p.outH * p.outW;
  float* out = dx + planeIn + (size_t)w0 * p.H;

  // ---- this thread's outputs: dzdy into registers, (column, row) by increments
  float dv[OPT];
  int oRow[OPT], oCol[OPT];
  {
    const float* src = dy + planeOut + (size_t)owLo * p.outH;
    int owr, oh;
    p.byOutH.divmod(tid, &owr, &oh);
    const int stepQ = p.outStepQ, stepR = p.outStepR;
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      const int o = tid + 256 * k;
      dv[k] = o < nOut ? src[o] : 0.f;
      oRow[k] = oh;
      oCol[k] = o < nOut ? owr : -1;
      owr += stepQ;
      oh += stepR;
      if (oh >= p.outH) {
        oh -= p.outH;
        ++owr;
      }
    }
  }

  // ---- accumulators
  if (p.accumulate) {
    stage<VEC4>(acc, out, nIn, tid);
  } else if (VEC4) {
    for (int i = tid; i < nIn / 4; i += 256) ((float4*)acc)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    for (int i = tid; i < nIn; i += 256) acc[i] = 0.f;
  }

  // ---- framed x: interior copied from the contiguous run of image columns [ca, cb), border cells = -inf
  if (MAX) {
    const int ca = max(cLo, 0), cb = min(cLo + nC, p.W);  // image columns present in the frame
    const float* src = x + planeIn + (size_t)ca * p.H;
    float* dst = xs + (ca - cLo) * Hp + p.pt;              // frame address of image element (row 0, column ca)
    if (VEC4) {
      const int HQ = p.byStageRow.d, n4 = (cb - ca) * HQ;
      int c, q;
      p.byStageRow.divmod(tid, &c, &q);
      const int stepQ = p.stageStepQ, stepR = p.stageStepR;
      for (int base = 0; base < n4; base += 2 * 256) {
        float4 v[2];
        int at[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int i = base + u * 256 + tid;
          if (i < n4) v[u] = ((const float4*)src)[i];
          at[u] = c * Hp + q * 4;
          c += stepQ;
          q += stepR;
          if (q >= HQ) {
            q -= HQ;
            ++c;
          }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int i = base + u * 256 + tid;
          if (i < n4) {
            dst[at[u]] = v[u].x;
            dst[at[u] + 1] = v[u].y;
            dst[at[u] + 2] = v[u].z;
            dst[at[u] + 3] = v[u].w;
          }
        }
      }
    } else {
      const int n = (cb - ca) * p.H;
      int c, h;
      p.byStageRow.divmod(tid, &c, &h);
      const int stepQ = p.stageStepQ, stepR = p.stageStepR;
      for (int i = tid; i < n; i += 256) {
        dst[c * Hp + h] = src[i];
        c += stepQ;
        h += stepR;
        if (h >= p.H) {
          h -= p.H;
          ++c;
        }
      }
    }
    // border cells (-inf): the rows above / below the image in every present column, one cell per thread ...
    const int below = max(Hp - p.pt - p.H, 0), nb = p.pt + below;
    if (nb > 0) {
      for (int i = tid; i < (cb - ca) * nb; i += 256) {
        int c, k;
        p.byBorder.divmod(i, &c, &k);
        xs[(ca - cLo + c) * Hp + (k < p.pt ? k : p.H + k)] = -INFINITY;
      }
    }
    // ... and whole columns left / right of the image
    for (int c = 0; c < ca - cLo; ++c)
      for (int r = tid; r < Hp; r += 256) xs[c * Hp + r] = -INFINITY;
    for (int c = cb - cLo; c < nC; ++c)
      for (int r = tid; r < Hp; r += 256) xs[c * Hp + r] = -INFINITY;
  }
  __syncthreads();

  if (MAX) {
    // ---- winner of each owned output and its rank among the outputs covering that winner
    int loc[OPT], rank[OPT];
    const int KH = p.KH;
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      loc[k] = -1;
      rank[k] = -1;
      if (oCol[k] >= 0) {
        const float* org = xs + (oCol[k] * p.sx) * Hp + oRow[k] * p.sy;  // window origin inside the frame
        float best = -INFINITY;
        int bj = -1, bi = 0, ra = 0, rb = 0;
        if (PH > 0 && PW > 0) {
          float v[PW > 0 ? PW : 1][PH > 0 ? PH : 1];
#pragma unroll
          for (int j = 0; j < PW; ++j)
#pragma unroll
            for (int i = 0; i < PH; ++i) v[j][i] = org[j * Hp + i];
#pragma unroll
          for (int j = 0; j < PW; ++j)
#pragma unroll
            for (int i = 0; i < PH; ++i)
              if (v[j][i] > best) {
                best = v[j][i];
                bj = j;
                bi = i;
                ra = p.rankH[i];
                rb = p.rankW[j];
              }
        } else {
          for (int j = 0; j < poolW; ++j)
            for (int i = 0; i < poolH; ++i) {
              const float v = org[j * Hp + i];
              if (v > best) {
                best = v;
                bj = j;
                bi = i;
                ra = p.rankH[i];
                rb = p.rankW[j];
              }
            }
        }
        if (bj >= 0) {
          const int w = cLo + oCol[k] * p.sx + bj - w0;  // tile-relative column of the winner
          if (w >= 0 && w < w1 - w0) {
            loc[k] = w * p.H + oRow[k] * p.sy + bi - p.pt;
            rank[k] = min(owLo + oCol[k], rb) * KH + min(oRow[k], ra);
          }
        }
      }
    }
    for (int t = 0; t < p.nPasses; ++t) {
#pragma unroll
      for (int k = 0; k < OPT; ++k)
        if (rank[k] == t) acc[loc[k]] = acc[loc[k]] + dv[k];
      __syncthreads();
    }
  } else {
    // ---- every owned output's share dzdy/area, then one pass per window position, last position first
    int hu[OPT], cu[OPT];
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      hu[k] = oRow[k] * p.sy - p.pt;
      cu[k] = (owLo + oCol[k]) * p.sx - p.pl;
      if (oCol[k] >= 0) {
        const int h2 = min(hu[k] + poolH, p.H), c2 = min(cu[k] + poolW, p.W);
        const int h1 = max(hu[k], 0), c1 = max(cu[k], 0);
        dv[k] = dv[k] * (1.0f / (float)((h2 - h1) * (c2 - c1)));  // derOutput * scale (bits/nnpooling.cu:68-96)
      }
      cu[k] -= w0;
    }
    for (int j = poolW - 1; j >= 0; --j)
      for (int i = poolH - 1; i >= 0; --i) {
#pragma unroll
        for (int k = 0; k < OPT; ++k) {
          const int w = cu[k] + j, h = hu[k] + i;
          if (oCol[k] >= 0 && (unsigned)w < (unsigned)(w1 - w0) && (unsigned)h < (unsigned)p.H) {
            const int idx = w * p.H + h;
            acc[idx] = acc[idx] + dv[k];
          }
        }
        __syncthreads();
      }
  }

  // ---- stream the accumulators out
  if (VEC4) {
    for (int i = tid; i < nIn / 4; i += 256) stream_store4((float4*)out + i, ((const float4*)acc)[i]);
  } else {
    for (int i = tid; i < nIn; i += 256) out[i] = acc[i];
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

// Forward for the two down-sampling poolings networks use -- 3x3 windows, stride 2, one row / column of padding in
// front, and 2x2 windows, stride 2, no padding -- on planes whose height is a multiple of 4 and whose width is
// even.  A thread owns four input rows (16-byte loads), which hold both rows of two outputs (the 3x3 window's row
// above them comes from one more 4-byte load), and walks along the width keeping the column it shares with the
// next window in registers: 2 to 4 loads per pair of outputs instead of 18, all of them whole 16-byte accesses
// that neighbouring lanes make side by side.  Each output is still computed in the scan order of the loop above
// (columns ascending, rows ascending inside a column; the first maximum wins, NaN never does).
template <bool MAX, bool P3>
__global__ __launch_bounds__(256) void pool_forward_quads(float* __restrict__ y, const float* __restrict__ x, int H, int W,
                                                          int quads, int segments, int owPerSegment, unsigned total) {
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= total) return;
  const int j = (int)(idx % (unsigned)quads);
  const unsigned rest = idx / (unsigned)quads;
  const int seg = (int)(rest % (unsigned)segments);
  const size_t z = rest / (unsigned)segments;
  const int outH = H / 2, outW = W / 2;
  const float* xp = x + z * (size_t)H * W + 4 * j;
  float* yp = y + z * (size_t)outH * outW + 2 * j;
  const int ow0 = seg * owPerSegment, ow1 = min(ow0 + owPerSegment, outW);
  constexpr int ROWS = P3 ? 5 : 4;  // rows 4j-1 .. 4j+3 (3x3) or 4j .. 4j+3
  const bool top = P3 && j > 0;     // the row above the quad exists
  auto column = [&](int c, float (&v)[ROWS]) {
    const v4f q = *(const v4f*)(xp + (size_t)c * H);
    if (P3) {
      v[0] = top ? xp[(size_t)c * H - 1] : 0.f;
      v[1] = q.x; v[2] = q.y; v[3] = q.z; v[4] = q.w;
    } else {
      v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    }
  };
  float a[ROWS], b[ROWS], c[ROWS];
  // one output: rows [R0, R0 + N) of the columns a (only if useA), b, c, in scan order
  auto scan = [&](float& acc, const float (&col)[ROWS], int r0, int n) {
#pragma unroll
    for (int h = 0; h < 3; ++h)
      if (h < n) {
        const float v = col[r0 + h];
        if (MAX) acc = (acc < v) ? v : acc;
        else acc = acc + v;
      }
  };
  auto output = [&](bool useA, int r0, int n) -> float {
    float acc = MAX ? -INFINITY : 0.f;
    if (useA) scan(acc, a, r0, n);
    scan(acc, b, r0, n);
    scan(acc, c, r0, n);
    return MAX ? acc : acc * (1.0f / (float)(n * (useA ? 3 : 2)));
  };
  // The columns of the next pair of outputs are loaded before this pair is computed: twice the loads in flight per
  // thread (the walk along the width is a chain of small dependent steps otherwise).
  if (ow0 >= ow1) return;
  float bn[ROWS], cn[ROWS];
  if (P3) {
    bool haveA = ow0 > 0;
    if (haveA) column(2 * ow0 - 1, a);
    column(2 * ow0, b);
    column(2 * ow0 + 1, c);
    for (int ow = ow0; ow < ow1; ++ow) {
      const bool more = ow + 1 < ow1;
      if (more) {
        column(2 * ow + 2, bn);
        column(2 * ow + 3, cn);
      }
      float2 r;
      // output row 2j: rows 4j-1 .. 4j+1 (without the first when it is above the plane); row 2j+1: rows 4j+1 .. 4j+3
      if (haveA) {
        r.x = top ? output(true, 0, 3) : output(true, 1, 2);
        r.y = output(true, 2, 3);
      } else {
        r.x = top ? output(false, 0, 3) : output(false, 1, 2);
        r.y = output(false, 2, 3);
      }
      *(float2*)(yp + (size_t)ow * outH) = r;
#pragma unroll
      for (int k = 0; k < ROWS; ++k) {
        a[k] = c[k];
        b[k] = bn[k];
        c[k] = cn[k];
      }
      haveA = true;
    }
  } else {
    column(2 * ow0, b);
    column(2 * ow0 + 1, c);
    for (int ow = ow0; ow < ow1; ++ow) {
      const bool more = ow + 1 < ow1;
      if (more) {
        column(2 * ow + 2, bn);
        column(2 * ow + 3, cn);
      }
      float2 r;
      r.x = output(false, 0, 2);
      r.y = output(false, 2, 2);
      *(float2*)(yp + (size_t)ow * outH) = r;
#pragma unroll
      for (int k = 0; k < ROWS; ++k) {
        b[k] = bn[k];
        c[k] = cn[k];
      }
    }
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
  if ((long long)g->H * g->W >= (1ll << 31) || g->H >= 32768 || g->W >= 32768)
    return fail(MCN_UNSUPPORTED, "%s: planes larger than 32767 x 32767 are not supported", who);
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
  for (int i = 0; i < 8; ++i) {
    p->rankH[i] = i < g->poolH ? (g->poolH - 1 - i) / g->strideY : 0;
    p->rankW[i] = i < g->poolW ? (g->poolW - 1 - i) / g->strideX : 0;
  }
  return MCN_SUCCESS;
}

// LDS bytes the tiled kernel needs for tile width TW (maximum over the tiles of a plane).
size_t tile_lds_bytes(const PoolP& p, bool isMax, bool useFlags, int TW) {
  size_t worst = 0;
  for (int w0 = 0; w0 < p.W; w0 += TW) {
    const int w1 = std::min(w0 + TW, p.W);
    const int num = w0 + p.pl - p.poolW + 1;
    const int owLo = num <= 0 ? 0 : (num + p.sx - 1) / p.sx;
    const int owHi = std::min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);
    const int nOW = std::max(owHi - owLo + 1, 0);
    const int wa = std::max(owLo * p.sx - p.pl, 0);
    const int wb = nOW > 0 ? std::min(owHi * p.sx - p.pl + p.poolW, p.W) : wa;
    auto pad4 = [](size_t n) { return (n + 3) & ~(size_t)3; };
    size_t need = pad4((size_t)p.H) + pad4((size_t)TW) + pad4((size_t)nOW * p.outH);
    if (isMax) need += pad4((size_t)(wb - wa) * p.H) + (useFlags ? pad4((size_t)(w1 - w0) * p.H) : pad4((size_t)nOW * p.outH));
    worst = std::max(worst, need * sizeof(float));
  }
  return worst;
}

}  // namespace

// the double-precision entry of the kernel above (f64.hip)
bool pool_avg_backward_tiles_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, double* derInput,
                                    const double* derOutput, int accumulate) {
  return avg_tiles_launch<double>(s, g, outH, outW, derInput, derOutput, accumulate);
}

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
  // the down-sampling poolings of the usual networks: four input rows per thread
  {
    const bool p3 = p.poolH == 3 && p.poolW == 3 && p.pt == 1 && p.pl == 1;
    const bool p2 = p.poolH == 2 && p.poolW == 2 && p.pt == 0 && p.pl == 0;
    if ((p3 || p2) && p.sy == 2 && p.sx == 2 && p.H % 4 == 0 && p.W % 2 == 0 && p.outH == p.H / 2 && p.outW == p.W / 2 &&
        aligned16(x) && aligned16(y) && !tunable("pool_force_gather", 0)) {
      const int quads = p.H / 4;
      const size_t planes = (size_t)g->C * g->N;
      // many short walks beat few long ones (measured: 2 output columns per thread 26 us, 14 per thread 32 us on
      // 112x112x64x32): enough threads for 8 wavefronts per SIMD, each with at least two output columns
      const size_t wantThreads = (size_t)2048 * 1024;
      int segments = (int)std::min<size_t>(std::max<size_t>(1, (wantThreads + planes * quads - 1) / (planes * quads)),
                                           (size_t)std::max(1, p.outW / 2));
      const int owPerSegment = (p.outW + segments - 1) / segments;
      segments = (p.outW + owPerSegment - 1) / owPerSegment;
      const size_t threads = planes * quads * segments;
      if (threads < (1ull << 32)) {
        const dim3 grid((unsigned)((threads + 255) / 256));
        KernelTimer timer("pool_forward_quads", as_stream(stream));
#define MCN_POOL_QUADS(MAXF, P3F)                                                                                  \
  hipLaunchKernelGGL((pool_forward_quads<MAXF, P3F>), grid, dim3(256), 0, as_stream(stream), y, x, p.H, p.W, quads, \
                     segments, owPerSegment, (unsigned)threads)
        if (g->method == MCN_POOL_MAX) { if (p3) MCN_POOL_QUADS(true, true); else MCN_POOL_QUADS(true, false); }
        else { if (p3) MCN_POOL_QUADS(false, true); else MCN_POOL_QUADS(false, false); }
#undef MCN_POOL_QUADS
        return check_launch("mcn_pool_forward");
      }
    }
  }
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

  const size_t budget = (size_t)std::min(std::max(tunable("pool_lds_bytes", 16 * 1024), 1024), 64 * 1024);
  const int kh = (p.poolH + p.sy - 1) / p.sy, kw = (p.poolW + p.sx - 1) / p.sx;
  const int passes = isMax ? kh * kw : p.poolH * p.poolW;
  const bool vecIn = (p.H % 4 == 0) && aligned16(derInput);

  // ---- max pooling, 3x3 windows at stride 2 with padding 1 in front, plane height a multiple of 4
  if (isMax && pool_max_backward_pairs_launch(s, g, p.outH, p.outW, derInput, x, derOutput, accumulate))
    return check_launch("mcn_pool_backward");
  // ---- max pooling, plane height a multiple of 4: streaming kernel
  if (isMax && pool_max_backward_stream_launch(s, g, p.outH, p.outW, derInput, x, derOutput, accumulate))
    return check_launch("mcn_pool_backward");

  // ---- average over one window that covers the whole plane (the pooling before a network's classifier): every
  //      element receives its plane's dzdy / (H*W), the single contribution the general kernels would add
  if (!isMax && p.outH == 1 && p.outW == 1 && p.poolH - p.pt >= p.H && p.poolW - p.pl >= p.W && total < (1ull << 32) &&
      !tunable("pool_force_gather", 0)) {
    KernelTimer timer("pool_avg_backward_whole", s);
    hipLaunchKernelGGL(pool_avg_backward_whole, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, derInput, derOutput,
                       (unsigned)total, (unsigned)(p.H * p.W), p.accumulate);
    return check_launch("mcn_pool_backward");
  }

  // ---- average over windows that tile the plane exactly: one streaming pass in memory order
  if (avg_tiles_launch<float>(s, g, p.outH, p.outW, derInput, derOutput, accumulate)) return check_launch("mcn_pool_backward");

  // ---- ordered passes.  Widest tile whose LDS fits the budget and whose outputs fit 4 per thread.
  if (passes <= 16 && p.poolH <= 8 && p.poolW <= 8 && !tunable("pool_force_gather", 0)) {
    int tiles = 0, maxOut = 0;
    size_t lds = 0;
    for (int nT = 1; nT <= p.W; ++nT) {
      const int TW = (p.W + nT - 1) / nT;
      if (nT > 1 && TW == (p.W + nT - 2) / (nT - 1)) continue;
      size_t worst = 0;
      int worstOut = 0;
      for (int w0 = 0; w0 < p.W; w0 += TW) {
        const int w1 = std::min(w0 + TW, p.W);
        const int num = w0 + p.pl - p.poolW + 1;
        const int owLo = num <= 0 ? 0 : (num + p.sx - 1) / p.sx;
        const int owHi = std::min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);
        const int nOW = std::max(owHi - owLo + 1, 0);
        auto pad4 = [](size_t n) { return (n + 3) & ~(size_t)3; };
        size_t need = pad4((size_t)(w1 - w0) * p.H);
        if (isMax) {
          const size_t nC = nOW > 0 ? (size_t)(owHi - owLo) * p.sx + p.poolW : 0;
          const size_t Hp = (size_t)std::max((p.outH - 1) * p.sy + p.poolH, p.pt + p.H);
          need += nC * Hp;
        }
        worst = std::max(worst, need * sizeof(float));
        worstOut = std::max(worstOut, nOW * p.outH);
      }
      if (worst <= budget && worstOut <= 4 * 256) {
        tiles = (p.W + TW - 1) / TW;
        p.TW = TW;
        lds = worst;
        maxOut = worstOut;
        break;
      }
    }
    if (tiles > 0 && planes * tiles < (1ull << 31)) {
      p.tilesPerPlane = tiles;
      const int stageRow = vecIn ? p.H / 4 : p.H;
      p.byTiles = FastDiv(tiles);
      p.bySx = FastDiv(p.sx);
      p.byOutH = FastDiv(p.outH);
      p.byStageRow = FastDiv(stageRow);
      p.byBorder = FastDiv(std::max(p.pt + std::max((p.outH - 1) * p.sy + p.poolH - p.pt - p.H, 0), 1));  // = Hp - H
      p.outStepQ = 256 / p.outH;
      p.outStepR = 256 % p.outH;
      p.stageStepQ = 256 / stageRow;
      p.stageStepR = 256 % stageRow;
      p.KH = kh;
      p.nPasses = passes;
      const dim3 grid((unsigned)(planes * tiles)), block(256);
      KernelTimer timer("pool_backward_passes", s);
#define MCN_POOL_PASSES(MAXF, VECF, OPTF, PHF, PWF) \
  hipLaunchKernelGGL((pool_backward_passes<MAXF, VECF, OPTF, PHF, PWF>), grid, block, lds, s, derInput, x, derOutput, p)
#define MCN_POOL_SHAPE(MAXF, VECF, OPTF)                                                  \
  do {                                                                                    \
    if (p.poolH == 3 && p.poolW == 3) MCN_POOL_PASSES(MAXF, VECF, OPTF, 3, 3);             \
    else if (p.poolH == 2 && p.poolW == 2) MCN_POOL_PASSES(MAXF, VECF, OPTF, 2, 2);        \
    else MCN_POOL_PASSES(MAXF, VECF, OPTF, 0, 0);                                          \
  } while (0)
#define MCN_POOL_OPT(MAXF, VECF)                        \
  do {                                                  \
    if (maxOut <= 256) MCN_POOL_SHAPE(MAXF, VECF, 1);      \
    else if (maxOut <= 512) MCN_POOL_SHAPE(MAXF, VECF, 2); \
    else if (maxOut <= 768) MCN_POOL_SHAPE(MAXF, VECF, 3); \
    else MCN_POOL_SHAPE(MAXF, VECF, 4);                    \
  } while (0)
      if (isMax) {
        if (vecIn) MCN_POOL_OPT(true, true);
        else MCN_POOL_OPT(true, false);
      } else {
        if (vecIn) MCN_POOL_OPT(false, true);
        else MCN_POOL_OPT(false, false);
      }
#undef MCN_POOL_OPT
#undef MCN_POOL_SHAPE
#undef MCN_POOL_PASSES
      return check_launch("mcn_pool_backward");
    }
  }

  // ---- general tiled gather (any window / stride): widest tile whose staging fits the LDS budget
  const bool useFlags = isMax && kh <= 3 && kw <= 3;  // winners flagged by outputs; otherwise inputs poll outputs
  int tiles = 0;
  size_t lds = 0;
  for (int nT = 1; nT <= p.W; ++nT) {
    const int TW = (p.W + nT - 1) / nT;
    if (nT > 1 && TW == (p.W + nT - 2) / (nT - 1)) continue;  // same width as the previous candidate
    const size_t need = tile_lds_bytes(p, isMax, useFlags, TW);
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
#define MCN_POOL_LAUNCH(MAXF, VECF, KHF, KWF) \
  hipLaunchKernelGGL((pool_backward_tiled<MAXF, VECF, KHF, KWF>), grid, block, lds, s, derInput, x, derOutput, p)
#define MCN_POOL_PICK(MAXF, VECF)                                  \
  do {                                                             \
    if (kh == 1 && kw == 1) MCN_POOL_LAUNCH(MAXF, VECF, 1, 1);      \
    else if (kh <= 2 && kw <= 2) MCN_POOL_LAUNCH(MAXF, VECF, 2, 2); \
    else if (kh <= 3 && kw <= 3) MCN_POOL_LAUNCH(MAXF, VECF, 3, 3); \
    else MCN_POOL_LAUNCH(MAXF, VECF, 0, 0);                         \
  } while (0)
#define MCN_POOL_FLAGS(VECF)                                                                                       \
  do {                                                                                                           \
    if (p.poolH == 2 && p.poolW == 2 && kh == 1 && kw == 1)                                                      \
      hipLaunchKernelGGL((pool_max_backward_flags<VECF, 1, 1, 2, 2>), grid, block, lds, s, derInput, x, derOutput, p); \
    else if (p.poolH == 3 && p.poolW == 3 && kh == 2 && kw == 2)                                                 \
      hipLaunchKernelGGL((pool_max_backward_flags<VECF, 2, 2, 3, 3>), grid, block, lds, s, derInput, x, derOutput, p); \
    else if (p.poolH == 3 && p.poolW == 3)                                                                       \
      hipLaunchKernelGGL((pool_max_backward_flags<VECF, 3, 3, 3, 3>), grid, block, lds, s, derInput, x, derOutput, p); \
    else                                                                                                         \
      hipLaunchKernelGGL((pool_max_backward_flags<VECF, 3, 3, 0, 0>), grid, block, lds, s, derInput, x, derOutput, p); \
  } while (0)
    if (useFlags) {
      if (vec) MCN_POOL_FLAGS(true);
      else MCN_POOL_FLAGS(false);
    } else if (isMax) {
      if (vec) MCN_POOL_PICK(true, true);
      else MCN_POOL_PICK(true, false);
    } else {
      if (vec) MCN_POOL_PICK(false, true);
      else MCN_POOL_PICK(false, false);
    }
#undef MCN_POOL_PICK
#undef MCN_POOL_FLAGS
#undef MCN_POOL_LAUNCH
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
