// vl_nnloss on the device: the categorical losses (one label per prediction vector: classerror, topkerror, log,
// softmaxlog, mhinge, mshinge) and the attribute losses (one label per prediction scalar: binaryerror, binarylog,
// logistic, hinge), value and derivative (matlab/vl_nnloss.m:136-317; the reference evaluates these formulas with
// gpuArray arithmetic from MATLAB).  Tiny next to the rest of a network's step: the layout is chosen so that it is
// never a latency problem (a wavefront per prediction vector when there are few of them, e.g. 1 x 1 x 1000 x N
// class scores; a thread per vector when they are pixels of a map), not for bandwidth records.
#include "mcn_internal.hpp"

#include <algorithm>

#pragma clang fp contract(off)

namespace mcn {
namespace {

struct LossP {
  int HW, C, N;          // pixels per image, channels (classes / attributes), images
  int kind, topK;
  float threshold;
  int divide;            // N when normalised (the sum, or every derivative, is divided by it), else 0
  size_t nLabels;        // N (one label per image) or HW*N (categorical) / HW*C*N (attributes)
  size_t nWeights;       // 0, or the length of the instance weights, broadcast by index modulo
};

__device__ __forceinline__ float weight_of(const LossP& p, const float* __restrict__ w, size_t item, float label) {
  float v = label != 0.f ? 1.f : 0.f;          // null labels are skipped (vl_nnloss.m:183-197)
  if (w) v = v * w[item % p.nWeights];           // times the caller's instance weights, broadcast (:203-211)
  return v;
}

// reductions over the LANES lanes that share a prediction vector (1: nothing to do)
template <int LANES>
__device__ __forceinline__ float lanes_max(float v) {
  if (LANES > 1) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  }
  return v;
}
template <int LANES>
__device__ __forceinline__ float lanes_sum(float v) {
  if (LANES > 1) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  }
  return v;
}
template <int LANES>
__device__ __forceinline__ int lanes_sum(int v) {
  if (LANES > 1) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  }
  return v;
}
// the largest value and, among equals, the lowest index (MATLAB's max and stable descending sort)
template <int LANES>
__device__ __forceinline__ void lanes_argmax(float& v, int& i) {
  if (LANES > 1) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(v, o);
      const int oi = __shfl_xor(i, o);
      if (ov > v || (ov == v && oi < i)) {
        v = ov;
        i = oi;
      }
    }
  }
}

// One prediction vector (pixel q of image n) per LANES lanes.  BACKWARD = false: terms[item] = weight * t.
// BACKWARD = true: dzdx of the vector.
template <int LANES, bool BACKWARD>
__global__ __launch_bounds__(256) void loss_categorical(float* __restrict__ out, const float* __restrict__ x,
                                                        const float* __restrict__ labels, const float* __restrict__ weights,
                                                        float dzdy, LossP p, size_t items) {
  const size_t item = ((size_t)blockIdx.x * 256 + threadIdx.x) / LANES;
  const int lane = LANES > 1 ? (int)(threadIdx.x & (LANES - 1)) : 0;
  if (item >= items) return;   // (whole groups of LANES lanes leave together)
  const size_t n = item / p.HW, q = item - n * p.HW;
  const float* xv = x + n * (size_t)p.HW * p.C + q;      // channel c at xv[c * HW]
  const float label = labels[p.nLabels == (size_t)p.N ? n : item];
  const float w = weight_of(p, weights, item, label);
  // the label's channel; a null label addresses channel 0 like the reference's saturating uint64(c - 1) (:226)
  const int ci = label >= 1.f ? min((int)label - 1, p.C - 1) : 0;
  const float xc = xv[(size_t)ci * p.HW];

  float xmax = -__builtin_inff();
  int imax = 0x7fffffff;
  float qmax = -__builtin_inff();   // the same leaving the label's channel out (mshinge)
  int iq = 0x7fffffff;
  int above = 0;                    // channels ranked before the label's by a stable descending sort
#pragma unroll 8
  for (int c = lane; c < p.C; c += LANES) {
    const float v = xv[(size_t)c * p.HW];
    if (v > xmax) { xmax = v; imax = c; }
    if (c != ci && v > qmax) { qmax = v; iq = c; }
    above += (v > xc || (v == xc && c < ci)) ? 1 : 0;
  }
  lanes_argmax<LANES>(xmax, imax);
  lanes_argmax<LANES>(qmax, iq);
  above = lanes_sum<LANES>(above);
  float sumex = 0.f;
  if (p.kind == MCN_LOSS_SOFTMAXLOG) {
#pragma unroll 8
    for (int c = lane; c < p.C; c += LANES) sumex += expf(xv[(size_t)c * p.HW] - xmax);
    sumex = lanes_sum<LANES>(sumex);
  }

  if (!BACKWARD) {
    float t = 0.f;
    switch (p.kind) {
      case MCN_LOSS_CLASSERROR: t = label != (float)(imax + 1) ? 1.f : 0.f; break;                        // :232-234
      case MCN_LOSS_TOPKERROR: t = (label >= 1.f && above < p.topK) ? 0.f : 1.f; break;                   // :235-237
      case MCN_LOSS_LOG: t = -logf(xc); break;                                                            // :238-239
      case MCN_LOSS_SOFTMAXLOG: t = xmax + logf(sumex) - xc; break;                                       // :240-243
      case MCN_LOSS_MHINGE: t = fmaxf(0.f, 1.f - xc); break;                                              // :244-245
      case MCN_LOSS_MSHINGE: t = fmaxf(0.f, 1.f - xc + qmax); break;                                      // :246-249
    }
    if (lane == 0) out[item] = w * t;
    return;
  }
  const float dz = dzdy * w;   // :275-277
  float* ov = out + n * (size_t)p.HW * p.C + q;
#pragma unroll 8
  for (int c = lane; c < p.C; c += LANES) {
    float y = 0.f;
    switch (p.kind) {
      case MCN_LOSS_LOG: y = c == ci ? -dz / fmaxf(xc, 1e-8f) : 0.f; break;                               // :281-283
      case MCN_LOSS_SOFTMAXLOG: {                                                                          // :284-289
        y = expf(xv[(size_t)c * p.HW] - xmax) / sumex;
        if (c == ci) y = y - 1.f;
        y = dz * y;
        break;
      }
      case MCN_LOSS_MHINGE: y = c == ci ? -dz * (xc < 1.f ? 1.f : 0.f) : 0.f; break;                      // :290-292
      case MCN_LOSS_MSHINGE: {                                                                             // :293-301
        const float W = dz * (xc - qmax < 1.f ? 1.f : 0.f);
        y = c == ci ? -W : (c == iq ? W : 0.f);
        break;
      }
      default: break;   // the error counts have no derivative (:279-280)
    }
    if (p.divide) y = y / (float)p.divide;   // :313-315
    ov[(size_t)c * p.HW] = y;
  }
}

// vl_nnsoftmax (matlab/vl_nnsoftmax.m:20-28): y = exp(x - max) / sum over the channels; with dzdy:
// dzdx = y .* (dzdy - sum(dzdy .* y)).  One prediction vector per LANES lanes, like the losses.
template <int LANES, bool BACKWARD>
__global__ __launch_bounds__(256) void softmax_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ dzdy, int HW, int C, size_t items) {
  const size_t item = ((size_t)blockIdx.x * 256 + threadIdx.x) / LANES;
  const int lane = LANES > 1 ? (int)(threadIdx.x & (LANES - 1)) : 0;
  if (item >= items) return;
  const size_t n = item / HW, q = item - n * HW;
  const size_t base = n * (size_t)HW * C + q;
  float xmax = -__builtin_inff();
#pragma unroll 8
  for (int c = lane; c < C; c += LANES) xmax = fmaxf(xmax, x[base + (size_t)c * HW]);
  xmax = lanes_max<LANES>(xmax);
  float sumex = 0.f;
#pragma unroll 8
  for (int c = lane; c < C; c += LANES) sumex += expf(x[base + (size_t)c * HW] - xmax);
  sumex = lanes_sum<LANES>(sumex);
  float dot = 0.f;
  if (BACKWARD) {
#pragma unroll 8
    for (int c = lane; c < C; c += LANES) dot += dzdy[base + (size_t)c * HW] * (expf(x[base + (size_t)c * HW] - xmax) / sumex);
    dot = lanes_sum<LANES>(dot);
  }
#pragma unroll 8
  for (int c = lane; c < C; c += LANES) {
    const float y = expf(x[base + (size_t)c * HW] - xmax) / sumex;
    out[base + (size_t)c * HW] = BACKWARD ? y * (dzdy[base + (size_t)c * HW] - dot) : y;
  }
}

// attribute losses: one label per element
template <bool BACKWARD>
__global__ __launch_bounds__(256) void loss_binary(float* __restrict__ out, const float* __restrict__ x,
                                                   const float* __restrict__ labels, const float* __restrict__ weights,
                                                   float dzdy, LossP p, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const float c = labels[i], v = x[i];
  // the weights are laid out like one image's labels (H x W x C) or like all of them
  const float w = weight_of(p, weights, i, c);
  if (!BACKWARD) {
    float t = 0.f;
    switch (p.kind) {
      case MCN_LOSS_BINARYERROR: {                                                                         // :250-251
        const float d = v - p.threshold;
        const float s = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
        t = s != c ? 1.f : 0.f;
        break;
      }
      case MCN_LOSS_BINARYLOG: t = -logf(c * (v - 0.5f) + 0.5f); break;                                   // :252-253
      case MCN_LOSS_LOGISTIC: {                                                                            // :254-258
        const float a = -c * v, b = fmaxf(0.f, a);
        t = b + logf(expf(-b) + expf(a - b));
        break;
      }
      case MCN_LOSS_HINGE: t = fmaxf(0.f, 1.f - c * v); break;                                            // :259-260
    }
    out[i] = w * t;
    return;
  }
  const float dz = dzdy * w;
  float y = 0.f;
  switch (p.kind) {
    case MCN_LOSS_BINARYLOG: y = -dz / (v + (c - 1.f) * 0.5f); break;                                     // :304-305
    case MCN_LOSS_LOGISTIC: y = -dz * c / (1.f + expf(c * v)); break;                                     // :306-309
    case MCN_LOSS_HINGE: y = -dz * c * (c * v < 1.f ? 1.f : 0.f); break;                                  // :310-311
    default: break;
  }
  if (p.divide) y = y / (float)p.divide;
  out[i] = y;
}

// y = sum of the terms (one workgroup, fixed order, double accumulators), divided by N when normalised (:262-271)
__global__ __launch_bounds__(256) void loss_total(float* __restrict__ y, const float* __restrict__ terms, size_t n,
                                                  int divide) {
  __shared__ double lds[4];
  double acc = 0.0;
  for (size_t i = threadIdx.x; i < n; i += 256) acc += (double)terms[i];
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = (float)((lds[0] + lds[1]) + (lds[2] + lds[3]));
    if (divide) s = s / (float)divide;
    y[0] = s;
  }
}

bool categorical(int kind) { return kind >= MCN_LOSS_CLASSERROR && kind <= MCN_LOSS_MSHINGE; }

int setup(const char* who, const mcn_loss_geom* g, size_t nLabels, const float* weights, size_t nWeights, LossP* p,
          size_t* items) {
  if (!g) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null geometry", who);
  if (g->H < 0 || g->W < 0 || g->C < 0 || g->N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if (g->loss < MCN_LOSS_CLASSERROR || g->loss > MCN_LOSS_HINGE) return fail(MCN_ILLEGAL_ARGUMENT, "%s: Unknown loss %d.", who, g->loss);
  if ((long long)g->H * g->W >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: plane too large", who);
  p->HW = g->H * g->W; p->C = g->C; p->N = g->N;
  p->kind = g->loss; p->topK = g->topK; p->threshold = (float)g->threshold;
  p->divide = g->normalise ? g->N : 0;
  const size_t vectors = (size_t)p->HW * g->N;
  if (categorical(g->loss)) {
    *items = vectors;
    // one label per image, or one per prediction vector (vl_nnloss.m:149-154,176-177)
    if (nLabels != (size_t)g->N && nLabels != vectors)
      return fail(MCN_ILLEGAL_ARGUMENT, "%s: C has neither one label per image nor one per prediction vector", who);
  } else {
    *items = vectors * g->C;
    if (nLabels != *items) return fail(MCN_ILLEGAL_ARGUMENT, "%s: C does not have one label per prediction scalar", who);
  }
  p->nLabels = nLabels;
  p->nWeights = weights ? nWeights : 0;
  if (weights && (nWeights == 0 || *items % nWeights != 0))
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: the instance weights cannot be broadcast to the labels", who);
  return MCN_SUCCESS;
}

template <bool BACKWARD>
int launch_items(hipStream_t s, const char* who, float* out, const float* x, const float* labels, const float* weights,
                 float dzdy, const LossP& p, size_t items) {
  if (!categorical(p.kind)) {
    const size_t blocks = (items + 255) / 256;
    if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
    KernelTimer timer("loss_binary", s);
    hipLaunchKernelGGL(loss_binary<BACKWARD>, dim3((unsigned)blocks), dim3(256), 0, s, out, x, labels, weights, dzdy, p, items);
    return check_launch(who);
  }
  // few vectors (class scores of a batch): a wavefront each; many (a map of pixels): a thread each, coalesced
  const bool wide = items < 16384;
  const size_t threads = wide ? items * 64 : items;
  const size_t blocks = (threads + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
  KernelTimer timer("loss_categorical", s);
  if (wide)
    hipLaunchKernelGGL((loss_categorical<64, BACKWARD>), dim3((unsigned)blocks), dim3(256), 0, s, out, x, labels, weights, dzdy, p, items);
  else
    hipLaunchKernelGGL((loss_categorical<1, BACKWARD>), dim3((unsigned)blocks), dim3(256), 0, s, out, x, labels, weights, dzdy, p, items);
  return check_launch(who);
}

int softmax(const char* who, mcn_stream_t stream, float* out, const float* x, const float* dzdy, int H, int W, int C, int N) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if ((long long)H * W >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: plane too large", who);
  const size_t items = (size_t)H * W * N;
  if (items == 0 || C == 0) return MCN_SUCCESS;
  if (!out || !x) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  const bool wide = items < 16384;
  const size_t blocks = ((wide ? items * 64 : items) + 255) / 256;
  if (blocks >= (1ull << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
  hipStream_t s = as_stream(stream);
  KernelTimer timer("softmax_kernel", s);
  const dim3 grid((unsigned)blocks), block(256);
  if (dzdy) {
    if (wide) hipLaunchKernelGGL((softmax_kernel<64, true>), grid, block, 0, s, out, x, dzdy, H * W, C, items);
    else hipLaunchKernelGGL((softmax_kernel<1, true>), grid, block, 0, s, out, x, dzdy, H * W, C, items);
  } else {
    if (wide) hipLaunchKernelGGL((softmax_kernel<64, false>), grid, block, 0, s, out, x, dzdy, H * W, C, items);
    else hipLaunchKernelGGL((softmax_kernel<1, false>), grid, block, 0, s, out, x, dzdy, H * W, C, items);
  }
  return check_launch(who);
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

size_t mcn_loss_workspace_bytes(const mcn_loss_geom* g) {
  if (!g || g->H < 0 || g->W < 0 || g->C < 0 || g->N < 0) return 0;
  const size_t vectors = (size_t)g->H * g->W * g->N;
  return (g->loss >= MCN_LOSS_BINARYERROR ? vectors * g->C : vectors) * sizeof(float);
}

int mcn_loss_forward(mcn_stream_t stream, const mcn_loss_geom* g, float* y, const float* x, const float* labels,
                     size_t nLabels, const float* instanceWeights, size_t nWeights, void* workspace, size_t workspaceBytes) {
  LossP p;
  size_t items;
  int rc = setup("mcn_loss_forward", g, nLabels, instanceWeights, nWeights, &p, &items);
  if (rc) return rc;
  if (!y) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_loss_forward: null output");
  hipStream_t s = as_stream(stream);
  if (items != 0) {
    if (!x || !labels) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_loss_forward: null tensor");
    if (!workspace || workspaceBytes < items * sizeof(float))
      return fail(MCN_ILLEGAL_ARGUMENT, "mcn_loss_forward: workspace too small (%zu < %zu bytes)", workspaceBytes,
                  items * sizeof(float));
    rc = launch_items<false>(s, "mcn_loss_forward", (float*)workspace, x, labels, instanceWeights, 0.f, p, items);
    if (rc) return rc;
  }
  KernelTimer timer("loss_total", s);
  hipLaunchKernelGGL(loss_total, dim3(1), dim3(256), 0, s, y, (const float*)workspace, items, p.divide);
  return check_launch("mcn_loss_forward");
}

int mcn_loss_backward(mcn_stream_t stream, const mcn_loss_geom* g, float* derInput, const float* x, const float* labels,
                      size_t nLabels, const float* instanceWeights, size_t nWeights, double derOutput) {
  LossP p;
  size_t items;
  int rc = setup("mcn_loss_backward", g, nLabels, instanceWeights, nWeights, &p, &items);
  if (rc) return rc;
  if (items == 0 || g->C == 0) return MCN_SUCCESS;
  if (!derInput || !x || !labels) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_loss_backward: null tensor");
  return launch_items<true>(as_stream(stream), "mcn_loss_backward", derInput, x, labels, instanceWeights, (float)derOutput, p,
                            items);
}

int mcn_softmax_forward(mcn_stream_t stream, float* y, const float* x, int H, int W, int C, int N) {
  return softmax("mcn_softmax_forward", stream, y, x, nullptr, H, W, C, N);
}

int mcn_softmax_backward(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, int H, int W, int C,
                         int N) {
  if (!derOutput && (size_t)H * W * C * N != 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_softmax_backward: null tensor");
  return softmax("mcn_softmax_backward", stream, derInput, x, derOutput, H, W, C, N);
}

}  // extern "C"
