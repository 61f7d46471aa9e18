// Pixel-major products with at most four output channels: the input gradient of a network's first layer (RGB or
// grey-level images: dzdx has 3 or 1 channels; bits/nnconv.cu:247-277) and forward products with as few filters.
// The 32-channel tiles of the other matrix kernels would multiply 8 to 32 times more than is asked for.
//
// v_mfma_f32_4x4x1_16b_f32 multiplies sixteen independent 4x1 by 1x4 blocks: with lane = pixel, the A operand is
// the gathered value of the lane's pixel (one dword per lane straight from global memory, as in the
// weights-stationary kernel), the B operand is the reduction row's weights for channels 0..3 (lane l takes channel
// l % 4, the same in every block), and register v of lane l accumulates pixel 4*(l/4) + v, channel l % 4.  No
// multiply is wasted on channels that do not exist beyond the fourth.
//
// A workgroup is four wavefronts on the same 128 pixels (two blocks of 64 per wavefront: a weight read from LDS
// feeds two multiplies); each wavefront takes a quarter of the gathered channels.  The taps
// go in groups of up to nine (the size that leaves the fewest empty slots: 3x3 -> 9, 5x5 -> 5, 4x4 -> 8, 7x7 -> 7):
// a wavefront works out its lanes' gather offsets (or "outside the image") once per group, then walks its
// channels with the group's taps innermost -- the loads of a channel fall into the same
// few cache lines (tap-outermost order sent every load of a 64-channel layer to L2: 32 waves per CU, each cycling
// through 64 planes, do not fit L1), and no address arithmetic is left beside the loads.  Each wavefront keeps its
// weights in LDS in that order; the four partial sums are added in a fixed order through LDS.
#include "conv_common.hpp"

#include <algorithm>

namespace mcn {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxTapGroup = 9;

struct FewP {
  unsigned inBytes;   // extent of the gathered tensor (buffer descriptor)
  int nGroups;        // tap groups: ceil(T / group size)
  int maxC;           // most channels a wavefront gets: ceil(Cin / 4)
  int tapMajor;       // row order of the packed bank (see conv_pack_weights)
  FastDiv byFH;
};

template <int kTapGroup>
__global__ __launch_bounds__(256, 2) void conv_few_mfma(float* __restrict__ out, const float* __restrict__ in,
                                                     const float* __restrict__ wt, const float* __restrict__ bias, PixP p,
                                                     FewP w) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int perWave = w.nGroups * w.maxC * kTapGroup * 4;
  float* wl = lds + wave * perWave;   // this wavefront's weights: [tap group][channel][tap in group][output channel 0..3]
  float* sums = lds + 4 * perWave;    // [wave][pixel block][register][lane]

  const int c0 = (p.Cin * wave) / 4, nC = (p.Cin * (wave + 1)) / 4 - c0;   // this wavefront's channels

  // ---- its weights, in the order it will walk them (taps past the last one: zeros); the 64 lanes take sixteen
  // (channel, tap) pairs x four output channels at a time
  {
    const int j = lane & 3, slot = lane >> 2;
    for (int tg = 0; tg < w.nGroups; ++tg) {
#pragma unroll 4
      for (int e0 = 0; e0 < nC * kTapGroup; e0 += 16) {
        const int e = e0 + slot;
        const int cc = e / kTapGroup, tt = e - cc * kTapGroup;
        const int t = tg * kTapGroup + tt, ci = c0 + cc;
        float v = 0.f;
        if (t < p.T && cc < nC) {
          const int bankRow = w.tapMajor ? ((ci >> 4) * 16 * p.T + t * 16 + (ci & 15)) : (t + p.T * ci);
          v = wt[(size_t)bankRow * p.coutPad + j];
        }
        if (cc < nC) wl[((tg * nC + cc) * kTapGroup + tt) * 4 + j] = v;
      }
    }
  }

  // ---- the lane's two pixels (workgroups numbered XCD by XCD: neighbours, whose taps reach into each other's
  // columns, sit behind the same L2)
  const int tile = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
  int ihB[2], iwB[2];
  unsigned voff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int m = tile * 128 + h * 64 + lane;
    const bool mvalid = m < p.M;
    int n, q, ow, oh;
    p.byQ.divmod(mvalid ? m : 0, &n, &q);
    p.byOH.divmod(q, &ow, &oh);
    ihB[h] = mvalid ? oh * p.sy : -0x40000000;  // (an idle lane fails every "row inside the image" test)
    iwB[h] = ow * p.sx;
    voff[h] = (unsigned)(n * p.inImg + oh * p.sy + p.IH * iwB[h]) * 4u;
  }
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, (int)w.inBytes, 0x00020000);
  const int planeBytes = p.IH * p.IW * 4;

  floatx4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int tg = 0; tg < w.nGroups; ++tg) {
    unsigned vo[2][kTapGroup];
#pragma unroll
    for (int tt = 0; tt < kTapGroup; ++tt) {
      const int t = tg * kTapGroup + tt;
      int j, i;
      w.byFH.divmod(t, &j, &i);
      const int dh = p.dhBase + i * p.dhStep, dw = p.dwBase + j * p.dwStep;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool ok = t < p.T && (unsigned)(ihB[h] + dh) < (unsigned)p.IH && (unsigned)(iwB[h] + dw) < (unsigned)p.IW;
        vo[h][tt] = ok ? voff[h] + (unsigned)((dh + p.IH * dw) * 4) : kOutside;
      }
    }
    const float* wg = wl + tg * nC * (kTapGroup * 4) + (lane & 3);
    for (int cc = 0; cc < nC; ++cc) {
      const int soff = (c0 + cc) * planeBytes;
      float a[2][kTapGroup];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int tt = 0; tt < kTapGroup; ++tt)
          a[h][tt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)vo[h][tt], soff, 0));
#pragma unroll
      for (int tt = 0; tt < kTapGroup; ++tt) {
        const float b = wg[(cc * kTapGroup + tt) * 4];
        acc[0] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[0][tt], b, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[1][tt], b, acc[1], 0, 0, 0);
      }
    }
  }

  // ---- the four partial sums, added in wavefront order by the first wavefront
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int v = 0; v < 4; ++v) sums[((wave * 2 + h) * 4 + v) * 64 + lane] = acc[h][v];
  __syncthreads();
  if (wave != 0) return;
  const int co = lane & 3;
  if (co >= p.Cout) return;
  const float bv = bias ? bias[co] : 0.f;
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int e = (h * 4 + v) * 64 + lane;
      const float s = ((sums[e] + sums[e + 512]) + sums[e + 1024]) + sums[e + 1536];
      const int mo = tile * 128 + h * 64 + (lane & ~3) + v;
      if (mo >= p.M) continue;
      int no, qo;
      p.byQ.divmod(mo, &no, &qo);
      float* o = out + (size_t)no * p.outImg + (size_t)co * p.outPlane + out_pixel_offset(p, qo);
      float r = p.alpha * s;
      if (p.beta != 0.f) r = fmaf(p.beta, *o, r);
      if (bias) r += bv;
      *o = r;
    }
}

}  // namespace

int conv_few_launch(hipStream_t s, const char* who, float* out, const float* in, const float* wt, const float* bias,
                    const PixP& p, bool tapMajor, int* handled) {
  *handled = 0;
  if (tunable("conv_no_few", 0)) return MCN_SUCCESS;
  if (p.Cout > 4 || p.coutPad < 4 || p.R < 1 || p.M < 1) return MCN_SUCCESS;
  const long long inBytes = ((long long)(p.N - 1) * p.inImg + (long long)p.Cin * p.IH * p.IW) * 4;
  if (inBytes >= (long long)kOutside) return MCN_SUCCESS;
  FewP w;
  w.inBytes = (unsigned)inBytes;
  // the group size: few empty slots (taps padded to whole groups), but not tiny groups (few loads in flight)
  int group = 1;
  double best = 1e30;
  for (int g = 1; g <= kMaxTapGroup; ++g) {
    const double score = (double)((p.T + g - 1) / g * g) * (1.0 + 0.5 / g);
    if (score < best) {
      best = score;
      group = g;
    }
  }
  w.nGroups = (p.T + group - 1) / group;
  w.maxC = (p.Cin + 3) / 4;
  w.tapMajor = tapMajor ? 1 : 0;
  w.byFH = FastDiv(p.FH);
  const size_t lds = ((size_t)4 * w.nGroups * w.maxC * group * 4 + 4 * 2 * 4 * 64) * sizeof(float);
  if (lds > 60 * 1024) return MCN_SUCCESS;  // long reductions stay with the tiled kernel
  const long long blocks = ((long long)p.M + 127) / 128;
  if (blocks >= (1ll << 31)) return MCN_SUCCESS;
  KernelTimer timer("conv_few_mfma", s);
#define MCN_FEW(G) \
  case G: hipLaunchKernelGGL(conv_few_mfma<G>, dim3((unsigned)blocks), dim3(256), lds, s, out, in, wt, bias, p, w); break
  switch (group) {
    MCN_FEW(1); MCN_FEW(2); MCN_FEW(3); MCN_FEW(4); MCN_FEW(5); MCN_FEW(6); MCN_FEW(7); MCN_FEW(8); MCN_FEW(9);
  }
#undef MCN_FEW
  *handled = 1;
  return check_launch(who);
}

}  // namespace mcn
