// Batch normalisation forward / backward for gfx950.
//
// Two launches per call:
//   1. bnorm_sums  -- grid (channel, image-group).  Each workgroup streams its planes of x (and dzdy)
//      once with 16-byte loads, widens every element to fp64 and keeps fp64 running sums per lane (the
//      kernel waits on memory, the fp64 arithmetic is hidden), reduces across the wavefront with shuffles and
//      across wavefronts through LDS, and writes one fp64 partial per (channel, group): sum x, sum x^2,
//      sum x*dzdy, sum dzdy.
//   2. bnorm_apply -- same grid.  Each workgroup re-reduces its channel's partials in a fixed order
//      (deterministic), derives mean / sigma / dzdg / dzdb in fp64 exactly as the reference formulas
//      (bits/nnbnorm.cu:101-164), and streams the elementwise result
//      dzdx = G1*(dzdy - dzdb/m) - G2*(x - mean), written as two fused multiply-adds.
//      The first group of each channel also stores dzdg, dzdb and the moments.
//   The apply pass can walk the planes in the reverse order of the sums pass so that it starts on the
//   data most recently pulled through the caches.
//
// Accuracy: the reference sums ~1e5 terms sequentially in the data type.  Here every product and every sum is
// fp64 (the inputs are float, so each product is exact), which puts the results next to the reference's own
// double-precision instantiation run on the same float data -- also where the one-pass variance
// E[x^2] - mean^2 cancels many digits (a constant channel, a channel with |mean| >> sigma), where a float
// accumulation -- the reference's included -- keeps nothing of the variance.
#include "mcn_internal.hpp"

#include <algorithm>
#include <atomic>

// Partial sums of mcn_bnorm_backward_static, the entry point that allocates nothing: one copy per device, held
// from the moment the library is loaded until the process ends.  In host code this name only identifies the
// symbol; the address kernels are given is looked up once per device (static_scratch below).
static __device__ __align__(256) unsigned char scratch[MCN_BNORM_STATIC_SCRATCH_BYTES];

namespace mcn {
namespace {

// Device address of `scratch` on the current device (every device has its own copy at its own address).
std::atomic<void*> g_scratch_address[kMaxDevices];

int static_scratch(const char* who, void** address) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(MCN_DEVICE_ERROR, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices) return fail(MCN_UNSUPPORTED, "%s: device ordinal %d is not supported", who, device);
  void* p = g_scratch_address[device].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return fail(MCN_DEVICE_ERROR, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
    }
    g_scratch_address[device].store(p, std::memory_order_release);
  }
  *address = p;
  return MCN_SUCCESS;
}

struct BnormP {
  int WH, C, N;
  int groups;        // image groups per channel (grid = C * groups)
  int reverse;       // apply pass walks logical ids backwards
  int teamShift[2];  // log2 of the threads that share one plane, for scalar [0] and 16-byte [1] accesses: planes
                     // smaller than a workgroup's 256 accesses are walked several at a time, one per team
  int oneLaunch;     // groups == 1 and the apply kernels compute the sums themselves (small channels): no sums launch
  int walk;                  // order of the workgroups: 1 by plane address, 0 channel-major XCD by XCD, 2 by plane address XCD by XCD
  int sumGroups, sumStride;  // the partial sums the apply kernels add up: sumGroups per channel, sumStride doubles each
                             // (groups and 4 after a sums launch of this file; 2 when a convolution summed its output)
  double mass;       // WH * N
  double epsilon;
};

__device__ __forceinline__ void image_range(const BnormP& p, int grp, int* n0, int* n1) {
  *n0 = (int)(((long long)p.N * grp) / p.groups);
  *n1 = (int)(((long long)p.N * (grp + 1)) / p.groups);
}

// y = a*(x - s) + k with the rounding of the forward pass: the moments as stored (float), everything else in
// double, the coefficients rounded to float once.  s is the mean rounded to float, taken off x first (as the
// reference's (x - mean)*coef + b does, bits/nnbnorm.cu:190-199): with a channel whose mean is large against its
// sigma, a*x and k would be two huge numbers that cancel.  k carries what the rounding of the mean left over.
// Forward and the ReLU-masked backward both go through here, so that "a*(x - s) + k > 0" decides the same way in both.
__device__ __forceinline__ void forward_coefficients(double mean, double sigma, float mult, float bias, float* a, float* k,
                                                     float* s) {
  const double coef = (double)mult / sigma;
  *s = (float)mean;
  *a = (float)coef;
  *k = (float)((double)bias - coef * (mean - (double)*s));
}

// One bit per element of a tensor, in element order: bit e % 32 of word e / 32 says "the ReLU behind this element let
// it through" (its output was > 0).  Written by the forward pass that applies that ReLU (stream_forward), read by the
// backward passes instead of the ReLU's output: a thirty-second of the bytes.  Planes must be whole words (W*H a
// multiple of 32).  The four bits of the 16-byte cell at element e (a multiple of 4):
__device__ __forceinline__ unsigned mask_nibble(const unsigned* __restrict__ bits, size_t e) {
  return (bits[e >> 5] >> (unsigned)(e & 31)) & 15u;
}
// dy where the bit is set, else dy*0 like mcn_relu_backward (a NaN or infinity stays visible)
__device__ __forceinline__ float4 mask_by_nibble(float4 d, unsigned nb) {
  return make_float4((nb & 1u) ? d.x : d.x * 0.f, (nb & 2u) ? d.y : d.y * 0.f, (nb & 4u) ? d.z : d.z * 0.f,
                     (nb & 8u) ? d.w : d.w * 0.f);
}

// Block-wide sum of NV doubles held per thread; result valid in thread 0.
template <int NV>
__device__ __forceinline__ void block_sum(double (&v)[NV], double* lds /* [4][NV] */) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = wave_sum(v[i]);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) lds[wave * NV + i] = v[i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = (lds[i] + lds[NV + i]) + (lds[2 * NV + i] + lds[3 * NV + i]);
  }
}

// MODE 0: sum x, sum x^2               (forward, moments from the batch)
// MODE 1: sum x*dy, sum dy             (backward, moments given)
// MODE 2: all four                     (backward, moments from the batch)
// RELU (MODE 1 only): dy is the derivative after a ReLU that followed this layer; it counts only where the
// layer's output a*x + k was positive (a, k: the forward pass's own coefficients, see forward_coefficients).
// YMASK (MODE 1 only): dy first passes the derivative of a ReLU whose *output* is ymask (dy counts where
// ymask > 0, else dy*0 like mcn_relu_backward), and the masked derivative is also written to `masked` for the
// passes that follow (this layer's apply pass, and whoever else consumes it).
// BITS (MODE 1, 16-byte accesses only): like YMASK, but the mask comes as one bit per element (`ymask` points at the
// words, see mask_nibble) and nothing is written.
template <int MODE, bool VEC4, bool RELU, bool YMASK, bool BITS = false>
__device__ __forceinline__ void sums_of_planes(double (&acc)[4], const float* __restrict__ x, const float* __restrict__ dy,
                                               const BnormP& p, int c, int n0, int n1, float ra, float rk, float rs,
                                               const float* __restrict__ ymask, float* __restrict__ masked, double* lds) {
  static_assert(!BITS || (VEC4 && MODE == 1 && !RELU && !YMASK), "the bit mask goes with 16-byte accesses and given moments");
  auto gate = [&](float xv, float dv) -> float { return RELU ? (fmaf(ra, xv - rs, rk) > 0.f ? dv : 0.f) : dv; };
  acc[0] = acc[1] = acc[2] = acc[3] = 0.0;
  const int shift = p.teamShift[VEC4 ? 1 : 0], TS = 1 << shift, teams = 256 >> shift;
  const int team = threadIdx.x >> shift, j0 = threadIdx.x & (TS - 1);
  for (int n = n0 + team; n < n1; n += teams) {
    const size_t base = (size_t)p.WH * (c + (size_t)p.C * n);
    if (VEC4) {
      const float4* x4 = (const float4*)(x + base);
      const float4* d4 = (const float4*)(MODE != 0 ? dy + base : x + base);
      for (int i = j0; i < p.WH / 4; i += TS) {
        const float4 a = x4[i];
        const double ax = (double)a.x, ay = (double)a.y, az = (double)a.z, aw = (double)a.w;
        if (MODE != 1) {
          acc[0] += (ax + ay) + (az + aw);
          acc[1] += fma(ax, ax, ay * ay) + fma(az, az, aw * aw);
        }
        if (MODE != 0) {
          float4 d = d4[i];
          if (RELU) d = make_float4(gate(a.x, d.x), gate(a.y, d.y), gate(a.z, d.z), gate(a.w, d.w));
          if (YMASK) {
            const float4 m = ((const float4*)(ymask + base))[i];
            d = make_float4(m.x > 0.f ? d.x : d.x * 0.f, m.y > 0.f ? d.y : d.y * 0.f, m.z > 0.f ? d.z : d.z * 0.f,
                            m.w > 0.f ? d.w : d.w * 0.f);
            ((float4*)(masked + base))[i] = d;
          }
          if (BITS) d = mask_by_nibble(d, mask_nibble((const unsigned*)ymask, base + 4 * (size_t)i));
          const double dx_ = (double)d.x, dy_ = (double)d.y, dz_ = (double)d.z, dw_ = (double)d.w;
          acc[2] += fma(ax, dx_, ay * dy_) + fma(az, dz_, aw * dw_);
          acc[3] += (dx_ + dy_) + (dz_ + dw_);
        }
      }
    } else {
      // four scalar loads of each tensor in flight per thread (lanes past the plane's end re-read its last element and
      // count it as zero)
      for (int i = j0; i < p.WH; i += 4 * TS) {
        float a[4], d[4], m[4];
        bool in[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          in[u] = i + u * TS < p.WH;
          const size_t at = base + (in[u] ? i + u * TS : p.WH - 1);
          a[u] = x[at];
          if (MODE != 0) d[u] = dy[at];
          if (YMASK) m[u] = ymask[at];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const double ad = in[u] ? (double)a[u] : 0.0;
          if (MODE != 1) {
            acc[0] += ad;
            acc[1] = fma(ad, ad, acc[1]);
          }
          if (MODE != 0) {
            float dv = gate(a[u], d[u]);
            if (YMASK) {
              dv = m[u] > 0.f ? dv : dv * 0.f;
              if (in[u]) masked[base + i + u * TS] = dv;
            }
            const double dd = in[u] ? (double)dv : 0.0;
            acc[2] = fma(ad, dd, acc[2]);
            acc[3] += dd;
          }
        }
      }
    }
  }
  block_sum<4>(acc, lds);
}

template <int MODE, bool VEC4, bool RELU = false, bool YMASK = false, bool BITS = false>
__global__ __launch_bounds__(256) void bnorm_sums(const float* __restrict__ x,
                                                  const float* __restrict__ dy,
                                                  double* __restrict__ partials, BnormP p,
                                                  const float* __restrict__ moments = nullptr,
                                                  const float* __restrict__ mult = nullptr,
                                                  const float* __restrict__ bias = nullptr,
                                                  const float* __restrict__ ymask = nullptr,
                                                  float* __restrict__ masked = nullptr) {
  static_assert(!RELU || MODE == 1, "the ReLU mask needs the moments of the forward pass");
  static_assert(!YMASK || (MODE == 1 && !RELU), "one kind of mask at a time, with given moments");
  static_assert(!BITS || !YMASK, "one kind of mask at a time");
  __shared__ double lds[16];
  // Workgroups in the order of their planes in memory (image-major: neighbours in the grid read neighbouring planes):
  // the summing pass of 56x56x256x32 takes 39.4 us that way against 41.5 channel-major (whose concurrent workgroups
  // read planes a whole image apart), XCD by XCD or not; nothing is shared between planes, so no numbering by XCD.
  int c, grp;
  if (p.walk == 0) {
    const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
    c = logical / p.groups;
    grp = logical - c * p.groups;
  } else {
    const int logical = p.walk == 1 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
    grp = logical / p.C;
    c = logical - grp * p.C;
  }
  int n0, n1;
  image_range(p, grp, &n0, &n1);
  float ra = 0.f, rk = 0.f, rs = 0.f;
  if (RELU) forward_coefficients((double)moments[c], (double)moments[c + p.C], mult[c], bias[c], &ra, &rk, &rs);
  double acc[4];
  sums_of_planes<MODE, VEC4, RELU, YMASK, BITS>(acc, x, dy, p, c, n0, n1, ra, rk, rs, ymask, masked, lds);
  if (threadIdx.x == 0) {
    double* out = partials + ((size_t)c * p.groups + grp) * 4;
    out[0] = acc[0];
    out[1] = acc[1];
    out[2] = acc[2];
    out[3] = acc[3];
  }
}

// The totals of channel c when its single workgroup computes them itself (oneLaunch): the sums over all its
// planes, handed to every thread.  `lds`: 20 doubles.
template <int MODE, bool VEC4, bool RELU, bool YMASK>
__device__ __forceinline__ void own_totals(double (&tot)[4], const float* __restrict__ x, const float* __restrict__ dy,
                                           const BnormP& p, int c, float ra, float rk, float rs,
                                           const float* __restrict__ ymask, float* __restrict__ masked, double* lds) {
  double acc[4];
  sums_of_planes<MODE, VEC4, RELU, YMASK>(acc, x, dy, p, c, 0, p.N, ra, rk, rs, ymask, masked, lds);
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) lds[16 + i] = acc[i];
  }
  __syncthreads();  // (also orders the masked derivative written above before the apply pass reads it)
#pragma unroll
  for (int i = 0; i < 4; ++i) tot[i] = lds[16 + i];
}

// Sum of a channel's partials in a fixed order: lane i owns groups i, i+64, ...; then a wave tree.
// Every lane of wave 0 ends with the totals; other waves read them from LDS.  More than 64 partials (the sums a
// convolution left, one per workgroup of its launch) are shared by all four wavefronts, thread i owning groups i,
// i+256, ..., and the four wavefront sums are added in wavefront order: a quarter of the dependent loads.
// `lds`: 20 doubles.
__device__ __forceinline__ void channel_totals(const double* __restrict__ partials, const BnormP& p,
                                               int c, double* lds, double (&tot)[4]) {
  const bool wide = p.sumGroups > kWave;
  if (wide || threadIdx.x < kWave) {
    double v[4] = {0.0, 0.0, 0.0, 0.0};
    for (int g = threadIdx.x; g < p.sumGroups; g += wide ? 256 : kWave) {
      const double* in = partials + ((size_t)c * p.sumGroups + g) * p.sumStride;
      v[0] += in[0];
      v[1] += in[1];
      if (p.sumStride == 4) {
        v[2] += in[2];
        v[3] += in[3];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = wave_sum(v[i]);
    if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) lds[(threadIdx.x / kWave) * 4 + i] = v[i];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) tot[i] = wide ? ((lds[i] + lds[4 + i]) + lds[8 + i]) + lds[12 + i] : lds[i];
}

// out = a*(in1 - t) + b*(in2 - s) + k over this workgroup's planes (in2 optional)
// RELU: in1 counts only where ra*(in2 - rs) + rk > 0 (in1 = derivative after the ReLU, in2 = the layer's input)
// BITS: in1 counts only where its bit is set (see mask_nibble), else as in1*0
template <bool TWO, bool VEC4, bool RELU = false, bool BITS = false>
__device__ __forceinline__ void stream_planes(float* __restrict__ out, const float* __restrict__ in1,
                                              const float* __restrict__ in2, float a, float b, float k, float s,
                                              float t, const BnormP& p, int c, int n0, int n1, float ra = 0.f, float rk = 0.f,
                                              float rs = 0.f, const unsigned* __restrict__ bits = nullptr) {
  static_assert(!RELU || TWO, "the mask is computed from the second stream");
  static_assert(!BITS || (VEC4 && TWO && !RELU), "the bit mask goes with 16-byte accesses");
  auto gate = [&](float xv, float dv) -> float { return RELU ? (fmaf(ra, xv - rs, rk) > 0.f ? dv : 0.f) : dv; };
  const int shift = p.teamShift[VEC4 ? 1 : 0], TS = 1 << shift, teams = 256 >> shift;
  const int team = threadIdx.x >> shift, j0 = threadIdx.x & (TS - 1);
  for (int nn = n0 + team; nn < n1; nn += teams) {
    const int n = p.reverse ? (n1 - 1 - (nn - n0)) : nn;
    const size_t base = (size_t)p.WH * (c + (size_t)p.C * n);
    if (VEC4) {
      const float4* s1 = (const float4*)(in1 + base);
      const float4* s2 = (const float4*)(TWO ? in2 + base : in1 + base);
      float4* o4 = (float4*)(out + base);
      for (int i = j0; i < p.WH / 4; i += TS) {
        float4 u = stream_load4(s1 + i);
        if (BITS) u = mask_by_nibble(u, mask_nibble(bits, base + 4 * (size_t)i));
        float4 r;
        if (TWO) {
          const float4 v = stream_load4(s2 + i);
          r.x = fmaf(a, gate(v.x, u.x) - t, fmaf(b, v.x - s, k));
          r.y = fmaf(a, gate(v.y, u.y) - t, fmaf(b, v.y - s, k));
          r.z = fmaf(a, gate(v.z, u.z) - t, fmaf(b, v.z - s, k));
          r.w = fmaf(a, gate(v.w, u.w) - t, fmaf(b, v.w - s, k));
        } else {
          r.x = fmaf(a, u.x, k);
          r.y = fmaf(a, u.y, k);
          r.z = fmaf(a, u.z, k);
          r.w = fmaf(a, u.w, k);
        }
        stream_store4(o4 + i, r);
      }
    } else {
      for (int i = j0; i < p.WH; i += TS) {
        const float u = in1[base + i];
        out[base + i] = TWO ? fmaf(a, gate(in2[base + i], u) - t, fmaf(b, in2[base + i] - s, k)) : fmaf(a, u, k);
      }
    }
  }
}

// Backward apply.  GIVEN: mean/sigma come from `moments` (input); otherwise from the partial sums and
// `moments` (if non-null) is written.
// ONE: 0 = totals from the partials of a sums launch; 1 = this workgroup sums its channel itself first (oneLaunch);
// 2 = the same with the mask of a later ReLU (dy = the raw derivative, ymask that ReLU's output, masked = where the
// masked derivative goes: the apply pass then reads it back).
// BITS (GIVEN, ONE = 0): dy first passes a ReLU whose mask comes as one bit per element in `ymask` (see mask_nibble).
template <bool GIVEN, bool VEC4, bool RELU = false, int ONE = 0, bool BITS = false>
__global__ __launch_bounds__(256) void bnorm_backward_apply(float* __restrict__ dx,
                                                            float* __restrict__ dmult,
                                                            float* __restrict__ dbias,
                                                            float* __restrict__ moments,
                                                            const float* __restrict__ x,
                                                            const float* __restrict__ mult,
                                                            const float* __restrict__ dy,
                                                            const double* __restrict__ partials,
                                                            BnormP p, const float* __restrict__ bias = nullptr,
                                                            const float* __restrict__ ymask = nullptr,
                                                            float* __restrict__ masked = nullptr) {
  static_assert(!RELU || GIVEN, "the ReLU mask needs the moments of the forward pass");
  static_assert(ONE != 2 || (GIVEN && !RELU), "one kind of mask at a time, with given moments");
  static_assert(!BITS || (GIVEN && !RELU && ONE == 0 && VEC4), "the bit mask goes with given moments and a summing launch");
  __shared__ double lds[20];
  int logical = p.walk == 1 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
  if (p.reverse) logical = (int)gridDim.x - 1 - logical;
  int c, grp;
  if (p.walk == 0 || p.oneLaunch) {
    c = logical / p.groups;
    grp = logical - c * p.groups;
  } else {
    grp = logical / p.C;
    c = logical - grp * p.C;
  }
  double tot[4];
  if (ONE) {
    float sa = 0.f, sk = 0.f, ss = 0.f;
    if (RELU) forward_coefficients((double)moments[c], (double)moments[c + p.C], mult[c], bias[c], &sa, &sk, &ss);
    own_totals<GIVEN ? 1 : 2, VEC4, RELU, ONE == 2>(tot, x, dy, p, c, sa, sk, ss, ymask, masked, lds);
    if (ONE == 2) dy = masked;
  } else {
    channel_totals(partials, p, c, lds, tot);
  }

  double mean, sigma;
  if (GIVEN) {
    mean = (double)moments[c];
    sigma = (double)moments[c + p.C];
  } else {
    mean = tot[0] / p.mass;
    const double var = fmax(0.0, tot[1] / p.mass - mean * mean);
    sigma = sqrt(var + p.epsilon);
  }
  const double dB = tot[3];
  const double dG = (tot[2] - mean * dB) / sigma;
  const double muz = dB / p.mass;
  const double G1 = (double)mult[c] / sigma;
  const double G2 = G1 * dG / (p.mass * sigma);
  if (grp == 0 && threadIdx.x == 0) {
    dmult[c] = (float)dG;
    dbias[c] = (float)dB;
    if (!GIVEN && moments) {
      moments[c] = (float)mean;
      moments[c + p.C] = (float)sigma;
    }
  }
  // dzdx = G1*(dy - muz) - G2*(x - mean) = G1*(dy - t) + (-G2)*(x - s) + (G2*(mean - s) - G1*(muz - t)) with
  // s = float(mean), t = float(muz): both means come off before anything is scaled, as in bits/nnbnorm.cu:148-160
  // (scaled first, a channel whose mean is large against its spread would cancel two huge numbers); the constant
  // carries what their rounding to float left over
  int n0, n1;
  image_range(p, grp, &n0, &n1);
  float ra = 0.f, rk = 0.f, rs = 0.f;
  if (RELU) forward_coefficients(mean, sigma, mult[c], bias[c], &ra, &rk, &rs);
  const float shift = (float)mean, shiftDy = (float)muz;
  stream_planes<true, VEC4, RELU, BITS>(dx, dy, x, (float)G1, (float)(-G2),
                                        (float)(G2 * (mean - (double)shift) - G1 * (muz - (double)shiftDy)), shift, shiftDy, p, c,
                                        n0, n1, ra, rk, rs, (const unsigned*)ymask);
}

// out = act(a*(in - s) + k [+ res]) over this workgroup's planes: the forward apply with the element-wise layers
// that follow it folded in.  Each element goes through the same roundings as the separate kernels would
// give it: subtract, fma, then add, then max.
// BITS: also writes which elements the ReLU let through, one bit each (see mask_nibble): eight neighbouring lanes hold
// the 32 elements of one word (the host admits only planes of whole words walked by teams of at least 8 lanes).
template <bool RES, bool RELU, bool VEC4, bool BITS = false>
__device__ __forceinline__ void stream_forward(float* __restrict__ out, const float* __restrict__ in,
                                               const float* __restrict__ res, float a, float k, float s,
                                               const BnormP& p, int c, int n0, int n1, unsigned* __restrict__ bits = nullptr) {
  static_assert(!BITS || (RELU && VEC4), "the bit mask is the ReLU's, written with 16-byte accesses");
  auto one = [&](float u, float r) -> float {
    float v = fmaf(a, u - s, k);
    if (RES) v = v + r;
    if (RELU) v = v > 0.f ? v : 0.f;
    return v;
  };
  const int shift = p.teamShift[VEC4 ? 1 : 0], TS = 1 << shift, teams = 256 >> shift;
  const int team = threadIdx.x >> shift, j0 = threadIdx.x & (TS - 1);
  for (int nn = n0 + team; nn < n1; nn += teams) {
    const int n = p.reverse ? (n1 - 1 - (nn - n0)) : nn;
    const size_t base = (size_t)p.WH * (c + (size_t)p.C * n);
    if (VEC4) {
      const float4* s1 = (const float4*)(in + base);
      const float4* s2 = (const float4*)((RES ? res : in) + base);
      float4* o4 = (float4*)(out + base);
      for (int i = j0; i < p.WH / 4; i += TS) {
        const float4 u = stream_load4(s1 + i);
        float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
        if (RES) r = stream_load4(s2 + i);
        const float4 v = make_float4(one(u.x, r.x), one(u.y, r.y), one(u.z, r.z), one(u.w, r.w));
        stream_store4(o4 + i, v);
        if (BITS) {
          unsigned wd = ((v.x > 0.f ? 1u : 0u) | (v.y > 0.f ? 2u : 0u) | (v.z > 0.f ? 4u : 0u) | (v.w > 0.f ? 8u : 0u))
                        << (4 * (threadIdx.x & 7));
          wd |= (unsigned)__shfl_xor((int)wd, 1);
          wd |= (unsigned)__shfl_xor((int)wd, 2);
          wd |= (unsigned)__shfl_xor((int)wd, 4);
          if ((threadIdx.x & 7) == 0) bits[(base + 4 * (size_t)i) >> 5] = wd;
        }
      }
    } else {
      for (int i = j0; i < p.WH; i += TS) out[base + i] = one(in[base + i], RES ? res[base + i] : 0.f);
    }
  }
}

// Forward apply: y = (g/sigma)*(x - mean) + b  (bits/nnbnorm.cu:190-199), optionally followed by "+ residual"
// (matlab/+dagnn/Sum.m) and ReLU (matlab/vl_nnrelu.m) in the same pass.
template <bool GIVEN, bool VEC4, bool RES, bool RELU, bool ONE = false, bool BITS = false>
__global__ __launch_bounds__(256) void bnorm_forward_apply(float* __restrict__ y,
                                                           float* __restrict__ moments,
                                                           const float* __restrict__ x,
                                                           const float* __restrict__ mult,
                                                           const float* __restrict__ bias,
                                                           const float* __restrict__ residual,
                                                           const double* __restrict__ partials,
                                                           BnormP p, unsigned* __restrict__ maskBits = nullptr) {
  __shared__ double lds[20];
  int logical = p.walk == 1 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);
  if (p.reverse) logical = (int)gridDim.x - 1 - logical;
  int c, grp;
  if (p.walk == 0 || p.oneLaunch) {
    c = logical / p.groups;
    grp = logical - c * p.groups;
  } else {
    grp = logical / p.C;
    c = logical - grp * p.C;
  }
  double mean, sigma;
  if (GIVEN) {
    mean = (double)moments[c];
    sigma = (double)moments[c + p.C];
  } else {
    double tot[4];
    if (ONE) own_totals<0, VEC4, false, false>(tot, x, x, p, c, 0.f, 0.f, 0.f, nullptr, nullptr, lds);
    else channel_totals(partials, p, c, lds, tot);
    mean = tot[0] / p.mass;
    const double var = fmax(0.0, tot[1] / p.mass - mean * mean);
    sigma = sqrt(var + p.epsilon);
    if (grp == 0 && threadIdx.x == 0 && moments) {
      moments[c] = (float)mean;
      moments[c + p.C] = (float)sigma;
    }
    // normalise with the moments as they are stored (like the reference, whose moments are of the data type):
    // a later pass that is given them reproduces this one bit for bit
    mean = (double)(float)mean;
    sigma = (double)(float)sigma;
  }
  float a, k, shift;
  forward_coefficients(mean, sigma, mult[c], bias[c], &a, &k, &shift);
  int n0, n1;
  image_range(p, grp, &n0, &n1);
  stream_forward<RES, RELU, VEC4, BITS>(y, x, residual, a, k, shift, p, c, n0, n1, maskBits);
}

int image_groups(int WH, int N) {
  // one plane per workgroup unless planes are small; then enough planes to own ~bnorm_block_elems
  const int want = 4096;
  const int perBlock = std::max(1, want / std::max(WH, 1));
  return std::max(1, (N + perBlock - 1) / perBlock);
}

int setup(const char* who, int H, int W, int C, int N, double epsilon, BnormP* p) {
  if (H < 0 || W < 0 || C < 0 || N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if ((long long)H * W >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: plane too large", who);
  p->WH = H * W;
  p->C = C;
  p->N = N;
  p->groups = image_groups(p->WH, N);
  // small channels (the 14x14 and 7x7 layers of a network at a few dozen images): one workgroup per channel sums
  // and applies in the same launch; the second pass over the channel's few KB comes out of the caches
  p->oneLaunch = 0;
  if ((long long)p->WH * N <= tunable("bnorm_one_launch_elems", 8192) && C >= 128) {
    p->groups = 1;
    p->oneLaunch = 1;
  }
  p->reverse = 1;
  p->walk = 1;
  for (int v = 0; v < 2; ++v) {
    const int accesses = v ? p->WH / 4 : p->WH;  // per plane
    int shift = 4;                               // teams of 16 ... 256 threads
    while (shift < 8 && (1 << shift) < accesses) ++shift;
    p->teamShift[v] = shift;
  }
  p->sumGroups = p->groups;
  p->sumStride = 4;
  p->mass = (double)p->WH * (double)N;
  p->epsilon = epsilon;
  if ((long long)C * p->groups >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: too many channels", who);
  return MCN_SUCCESS;
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

size_t mcn_bnorm_workspace_bytes(int H, int W, int C, int N) {
  if (H <= 0 || W <= 0 || C <= 0 || N <= 0) return 0;
  return (size_t)C * image_groups(H * W, N) * 4 * sizeof(double);
}

int mcn_bnorm_forward_fused(mcn_stream_t stream, float* y, float* moments, const float* x, const float* multipliers,
                            const float* biases, const float* residual, int relu, int H, int W, int C, int N,
                            double epsilon, int givenMoments, void* workspace, size_t workspaceBytes) {
  BnormP p;
  int rc = setup("mcn_bnorm_forward", H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if ((size_t)p.WH * C * N == 0) return MCN_SUCCESS;
  if (!y || !x || !multipliers || !biases) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward: null tensor");
  if (givenMoments && !moments) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward: moments are required");
  hipStream_t s = as_stream(stream);
  const bool vec = (p.WH % 4 == 0) && aligned16(y) && aligned16(x) && (!residual || aligned16(residual));
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  double* partials = (double*)workspace;
  const bool one = p.oneLaunch && !givenMoments;
  if (!givenMoments && !one) {
    if (!workspace || workspaceBytes < mcn_bnorm_workspace_bytes(H, W, C, N))
      return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward: workspace too small");
    {
      KernelTimer timer("bnorm_sums", s);
      if (vec) hipLaunchKernelGGL((bnorm_sums<0, true>), grid, block, 0, s, x, x, partials, p);
      else hipLaunchKernelGGL((bnorm_sums<0, false>), grid, block, 0, s, x, x, partials, p);
    }
    if ((rc = check_launch("mcn_bnorm_forward(sums)"))) return rc;
  } else {
    p.reverse = 0;
  }
  KernelTimer timer("bnorm_forward_apply", s);
#define MCN_BN_FWD(GIVENF, VECF, RESF, RELUF)                                                                          \
  do {                                                                                                                  \
    if (!GIVENF && one)                                                                                                 \
      hipLaunchKernelGGL((bnorm_forward_apply<false, VECF, RESF, RELUF, true>), grid, block, 0, s, y, moments, x,       \
                         multipliers, biases, residual, partials, p);                                                   \
    else                                                                                                                \
      hipLaunchKernelGGL((bnorm_forward_apply<GIVENF, VECF, RESF, RELUF>), grid, block, 0, s, y, moments, x, multipliers, \
                         biases, residual, partials, p);                                                                \
  } while (0)
#define MCN_BN_FWD_EPI(GIVENF, VECF)                        \
  do {                                                      \
    if (residual && relu) MCN_BN_FWD(GIVENF, VECF, true, true);   \
    else if (residual) MCN_BN_FWD(GIVENF, VECF, true, false);     \
    else if (relu) MCN_BN_FWD(GIVENF, VECF, false, true);         \
    else MCN_BN_FWD(GIVENF, VECF, false, false);                  \
  } while (0)
  if (givenMoments) {
    if (vec) MCN_BN_FWD_EPI(true, true);
    else MCN_BN_FWD_EPI(true, false);
  } else {
    if (vec) MCN_BN_FWD_EPI(false, true);
    else MCN_BN_FWD_EPI(false, false);
  }
#undef MCN_BN_FWD_EPI
#undef MCN_BN_FWD
  return check_launch("mcn_bnorm_forward");
}

// Planes of whole 32-bit words, walked 16 bytes per lane by teams of at least 8 lanes: what the one-bit-per-element
// ReLU masks need (see mask_nibble).
static bool mask_bits_fit(const BnormP& p) { return p.WH % 32 == 0 && p.teamShift[1] >= 3; }

static int forward_from_sums(const char* who, mcn_stream_t stream, float* y, float* moments, const float* x,
                             const float* multipliers, const float* biases, const float* residual, int relu, int H, int W,
                             int C, int N, double epsilon, const double* sums, int sumGroups, unsigned* maskBits) {
  BnormP p;
  int rc = setup(who, H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if ((size_t)p.WH * C * N == 0) return MCN_SUCCESS;
  if (!y || !x || !multipliers || !biases || !sums) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  if (sumGroups <= 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: no partial sums", who);
  if (p.oneLaunch) {  // (the grid of the two-launch form: the sums are there already)
    p.oneLaunch = 0;
    p.groups = image_groups(p.WH, N);
  }
  p.sumGroups = sumGroups;
  p.sumStride = 2;
  p.reverse = 0;
  hipStream_t s = as_stream(stream);
  const bool vec = (p.WH % 4 == 0) && aligned16(y) && aligned16(x) && (!residual || aligned16(residual));
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  if (maskBits) {
    if (!relu || !vec || !mask_bits_fit(p))
      return fail(MCN_UNSUPPORTED, "%s: the bit mask needs a ReLU, 16-byte aligned tensors and planes of a multiple of 32 elements", who);
    KernelTimer timer("bnorm_forward_apply", s);
    if (residual) hipLaunchKernelGGL((bnorm_forward_apply<false, true, true, true, false, true>), grid, block, 0, s, y, moments, x, multipliers, biases, residual, sums, p, maskBits);
    else hipLaunchKernelGGL((bnorm_forward_apply<false, true, false, true, false, true>), grid, block, 0, s, y, moments, x, multipliers, biases, residual, sums, p, maskBits);
    return check_launch(who);
  }
  KernelTimer timer("bnorm_forward_apply", s);
#define MCN_BN_SUMS(VECF, RESF, RELUF) \
  hipLaunchKernelGGL((bnorm_forward_apply<false, VECF, RESF, RELUF>), grid, block, 0, s, y, moments, x, multipliers, biases, residual, sums, p)
#define MCN_BN_SUMS_EPI(VECF)                              \
  do {                                                     \
    if (residual && relu) MCN_BN_SUMS(VECF, true, true);   \
    else if (residual) MCN_BN_SUMS(VECF, true, false);     \
    else if (relu) MCN_BN_SUMS(VECF, false, true);         \
    else MCN_BN_SUMS(VECF, false, false);                  \
  } while (0)
  if (vec) MCN_BN_SUMS_EPI(true);
  else MCN_BN_SUMS_EPI(false);
#undef MCN_BN_SUMS_EPI
#undef MCN_BN_SUMS
  return check_launch(who);
}

int mcn_bnorm_forward_sums(mcn_stream_t stream, float* y, float* moments, const float* x, const float* multipliers,
                           const float* biases, const float* residual, int relu, int H, int W, int C, int N, double epsilon,
                           const double* sums, int sumGroups) {
  return forward_from_sums("mcn_bnorm_forward_sums", stream, y, moments, x, multipliers, biases, residual, relu, H, W, C, N,
                           epsilon, sums, sumGroups, nullptr);
}

int mcn_bnorm_mask_bits_supported(int H, int W, int C, int N) {
  BnormP p;
  if (setup("mcn_bnorm_mask_bits_supported", H, W, C, N, 1e-4, &p) || (size_t)p.WH * C * N == 0) return 0;
  return mask_bits_fit(p) && !p.oneLaunch ? 1 : 0;
}

int mcn_bnorm_forward_sums_mask(mcn_stream_t stream, float* y, unsigned* maskBits, float* moments, const float* x,
                                const float* multipliers, const float* biases, const float* residual, int H, int W, int C,
                                int N, double epsilon, const double* sums, int sumGroups) {
  if (!maskBits) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_forward_sums_mask: null mask");
  return forward_from_sums("mcn_bnorm_forward_sums_mask", stream, y, moments, x, multipliers, biases, residual, 1, H, W, C, N,
                           epsilon, sums, sumGroups, maskBits);
}

int mcn_bnorm_backward_bits(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                            const float* moments, const float* x, const float* multipliers, const float* derOutput,
                            const unsigned* maskBits, int H, int W, int C, int N, double epsilon, void* workspace,
                            size_t workspaceBytes) {
  BnormP p;
  int rc = setup("mcn_bnorm_backward_bits", H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if ((size_t)p.WH * C * N == 0) return MCN_SUCCESS;
  if (!derInput || !derMultipliers || !derBiases || !moments || !x || !multipliers || !derOutput || !maskBits)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_bits: null tensor");
  if (!mask_bits_fit(p) || p.oneLaunch || !aligned16(derInput) || !aligned16(x) || !aligned16(derOutput))
    return fail(MCN_UNSUPPORTED, "mcn_bnorm_backward_bits: the bit mask needs 16-byte aligned tensors and planes of a multiple "
                "of 32 elements (ask mcn_bnorm_mask_bits_supported)");
  if (!workspace || workspaceBytes < mcn_bnorm_workspace_bytes(H, W, C, N))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_bits: workspace too small");
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  double* partials = (double*)workspace;
  float* mom = const_cast<float*>(moments);  // (the kernels only write moments when they are not given)
  const float* bitsAsMask = (const float*)maskBits;
  {
    KernelTimer timer("bnorm_sums", s);
    hipLaunchKernelGGL((bnorm_sums<1, true, false, false, true>), grid, block, 0, s, x, derOutput, partials, p, nullptr, nullptr,
                       nullptr, bitsAsMask, nullptr);
  }
  if ((rc = check_launch("mcn_bnorm_backward_bits(sums)"))) return rc;
  KernelTimer timer("bnorm_backward_apply", s);
  hipLaunchKernelGGL((bnorm_backward_apply<true, true, false, 0, true>), grid, block, 0, s, derInput, derMultipliers, derBiases,
                     mom, x, multipliers, derOutput, partials, p, nullptr, bitsAsMask, nullptr);
  return check_launch("mcn_bnorm_backward_bits");
}

int mcn_bnorm_forward(mcn_stream_t stream, float* y, float* moments, const float* x, const float* multipliers,
                      const float* biases, int H, int W, int C, int N, double epsilon, int givenMoments,
                      void* workspace, size_t workspaceBytes) {
  return mcn_bnorm_forward_fused(stream, y, moments, x, multipliers, biases, NULL, 0, H, W, C, N, epsilon,
                                 givenMoments, workspace, workspaceBytes);
}

int mcn_bnorm_backward_relu(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                            const float* moments, const float* x, const float* multipliers, const float* biases,
                            const float* derOutput, int H, int W, int C, int N, double epsilon, void* workspace,
                            size_t workspaceBytes) {
  BnormP p;
  int rc = setup("mcn_bnorm_backward_relu", H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if (C == 0) return MCN_SUCCESS;
  if (!derMultipliers || !derBiases || !multipliers || !biases || !moments)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_relu: null parameter tensor");
  if ((size_t)p.WH * N == 0) {
    if ((rc = mcn_fill(stream, derMultipliers, 0.f, (size_t)C))) return rc;
    return mcn_fill(stream, derBiases, 0.f, (size_t)C);
  }
  if (!derInput || !x || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_relu: null tensor");
  if (!workspace || workspaceBytes < mcn_bnorm_workspace_bytes(H, W, C, N))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_relu: workspace too small");
  hipStream_t s = as_stream(stream);
  const bool vec = (p.WH % 4 == 0) && aligned16(derInput) && aligned16(x) && aligned16(derOutput);
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  double* partials = (double*)workspace;
  float* mom = const_cast<float*>(moments);  // (the kernels only write moments when they are not given)
  if (p.oneLaunch) {
    KernelTimer timer("bnorm_backward_apply", s);
    if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true, true, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, biases);
    else hipLaunchKernelGGL((bnorm_backward_apply<true, false, true, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, biases);
    return check_launch("mcn_bnorm_backward_relu");
  }
  {
    KernelTimer timer("bnorm_sums", s);
    if (vec) hipLaunchKernelGGL((bnorm_sums<1, true, true>), grid, block, 0, s, x, derOutput, partials, p, moments, multipliers, biases);
    else hipLaunchKernelGGL((bnorm_sums<1, false, true>), grid, block, 0, s, x, derOutput, partials, p, moments, multipliers, biases);
  }
  if ((rc = check_launch("mcn_bnorm_backward_relu(sums)"))) return rc;
  KernelTimer timer("bnorm_backward_apply", s);
  if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true, true>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, biases);
  else hipLaunchKernelGGL((bnorm_backward_apply<true, false, true>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, biases);
  return check_launch("mcn_bnorm_backward_relu");
}

int mcn_bnorm_backward_masked(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                              const float* moments, const float* x, const float* multipliers, const float* derOutput,
                              const float* maskSource, float* maskedDerOutput, int H, int W, int C, int N,
                              double epsilon, void* workspace, size_t workspaceBytes) {
  BnormP p;
  int rc = setup("mcn_bnorm_backward_masked", H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if (C == 0) return MCN_SUCCESS;
  if (!derMultipliers || !derBiases || !multipliers || !moments)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_masked: null parameter tensor");
  if ((size_t)p.WH * N == 0) {
    if ((rc = mcn_fill(stream, derMultipliers, 0.f, (size_t)C))) return rc;
    return mcn_fill(stream, derBiases, 0.f, (size_t)C);
  }
  if (!derInput || !x || !derOutput || !maskSource || !maskedDerOutput)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_masked: null tensor");
  if (!workspace || workspaceBytes < mcn_bnorm_workspace_bytes(H, W, C, N))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_bnorm_backward_masked: workspace too small");
  hipStream_t s = as_stream(stream);
  const bool vec = (p.WH % 4 == 0) && aligned16(derInput) && aligned16(x) && aligned16(derOutput) && aligned16(maskSource) &&
                   aligned16(maskedDerOutput);
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  double* partials = (double*)workspace;
  float* mom = const_cast<float*>(moments);  // (the kernels only write moments when they are not given)
  if (p.oneLaunch) {
    KernelTimer timer("bnorm_backward_apply", s);
    if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true, false, 2>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, nullptr, maskSource, maskedDerOutput);
    else hipLaunchKernelGGL((bnorm_backward_apply<true, false, false, 2>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, derOutput, partials, p, nullptr, maskSource, maskedDerOutput);
    return check_launch("mcn_bnorm_backward_masked");
  }
  {
    KernelTimer timer("bnorm_sums", s);
    if (vec) hipLaunchKernelGGL((bnorm_sums<1, true, false, true>), grid, block, 0, s, x, derOutput, partials, p, nullptr, nullptr, nullptr, maskSource, maskedDerOutput);
    else hipLaunchKernelGGL((bnorm_sums<1, false, false, true>), grid, block, 0, s, x, derOutput, partials, p, nullptr, nullptr, nullptr, maskSource, maskedDerOutput);
  }
  if ((rc = check_launch("mcn_bnorm_backward_masked(sums)"))) return rc;
  KernelTimer timer("bnorm_backward_apply", s);
  if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, maskedDerOutput, partials, p);
  else hipLaunchKernelGGL((bnorm_backward_apply<true, false>), grid, block, 0, s, derInput, derMultipliers, derBiases, mom, x, multipliers, maskedDerOutput, partials, p);
  return check_launch("mcn_bnorm_backward_masked");
}

// Both forms of mcn_bnorm_backward.  staticScratch: the partial sums go to the library's own device array instead of a
// workspace of the caller's.
static int bnorm_backward_any(const char* who, mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                              float* moments, const float* x, const float* multipliers, const float* derOutput, int H,
                              int W, int C, int N, double epsilon, int givenMoments, void* workspace,
                              size_t workspaceBytes, bool staticScratch) {
  BnormP p;
  int rc = setup(who, H, W, C, N, epsilon, &p);
  if (rc) return rc;
  if (C == 0) return MCN_SUCCESS;
  if (!derMultipliers || !derBiases || !multipliers) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null parameter tensor", who);
  if ((size_t)p.WH * N == 0) {
    // nothing to sum over: the reference leaves dzdg = 0/sigma-related garbage; define zeros
    if ((rc = mcn_fill(stream, derMultipliers, 0.f, (size_t)C))) return rc;
    return mcn_fill(stream, derBiases, 0.f, (size_t)C);
  }
  if (!derInput || !x || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null tensor", who);
  if (givenMoments && !moments) return fail(MCN_ILLEGAL_ARGUMENT, "%s: moments are required", who);
  const size_t need = mcn_bnorm_workspace_bytes(H, W, C, N);
  if (staticScratch) {
    if (need > (size_t)MCN_BNORM_STATIC_SCRATCH_BYTES)
      return fail(MCN_UNSUPPORTED, "%s: this shape needs %zu bytes of partial sums, the built-in scratch holds %zu; use "
                  "mcn_bnorm_backward with a workspace", who, need, (size_t)MCN_BNORM_STATIC_SCRATCH_BYTES);
    if ((rc = static_scratch(who, &workspace))) return rc;
  } else if (!workspace || workspaceBytes < need) {
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: workspace too small", who);
  }
  hipStream_t s = as_stream(stream);
  const bool vec = (p.WH % 4 == 0) && aligned16(derInput) && aligned16(x) && aligned16(derOutput);
  const dim3 grid((unsigned)(C * p.groups)), block(256);
  double* partials = (double*)workspace;
  if (p.oneLaunch) {
    KernelTimer timer("bnorm_backward_apply", s);
    if (givenMoments) {
      if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true, false, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
      else hipLaunchKernelGGL((bnorm_backward_apply<true, false, false, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
    } else {
      if (vec) hipLaunchKernelGGL((bnorm_backward_apply<false, true, false, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
      else hipLaunchKernelGGL((bnorm_backward_apply<false, false, false, 1>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
    }
    return check_launch(who);
  }
  {
    KernelTimer timer("bnorm_sums", s);
    if (givenMoments) {
      if (vec) hipLaunchKernelGGL((bnorm_sums<1, true>), grid, block, 0, s, x, derOutput, partials, p);
      else hipLaunchKernelGGL((bnorm_sums<1, false>), grid, block, 0, s, x, derOutput, partials, p);
    } else {
      if (vec) hipLaunchKernelGGL((bnorm_sums<2, true>), grid, block, 0, s, x, derOutput, partials, p);
      else hipLaunchKernelGGL((bnorm_sums<2, false>), grid, block, 0, s, x, derOutput, partials, p);
    }
  }
  if ((rc = check_launch(who))) return rc;
  KernelTimer timer("bnorm_backward_apply", s);
  if (givenMoments) {
    if (vec) hipLaunchKernelGGL((bnorm_backward_apply<true, true>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
    else hipLaunchKernelGGL((bnorm_backward_apply<true, false>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
  } else {
    if (vec) hipLaunchKernelGGL((bnorm_backward_apply<false, true>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
    else hipLaunchKernelGGL((bnorm_backward_apply<false, false>), grid, block, 0, s, derInput, derMultipliers, derBiases, moments, x, multipliers, derOutput, partials, p);
  }
  return check_launch(who);
}

int mcn_bnorm_backward(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases, float* moments,
                       const float* x, const float* multipliers, const float* derOutput, int H, int W, int C,
                       int N, double epsilon, int givenMoments, void* workspace, size_t workspaceBytes) {
  return bnorm_backward_any("mcn_bnorm_backward", stream, derInput, derMultipliers, derBiases, moments, x, multipliers,
                            derOutput, H, W, C, N, epsilon, givenMoments, workspace, workspaceBytes, false);
}

int mcn_bnorm_backward_static(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases, float* moments,
                              const float* x, const float* multipliers, const float* derOutput, int H, int W, int C,
                              int N, double epsilon, int givenMoments) {
  return bnorm_backward_any("mcn_bnorm_backward_static", stream, derInput, derMultipliers, derBiases, moments, x,
                            multipliers, derOutput, H, W, C, N, epsilon, givenMoments, nullptr, 0, true);
}

}  // extern "C"
