// Implicit-GEMM convolution on the fp32 matrix cores of gfx950 (v_mfma_f32_32x32x2_f32), filter groups = 1.
//
// No im2row buffer exists anywhere: the gather of shifted, zero-padded pixels happens while tiles are
// loaded from global memory into LDS.
//
// Two kernels:
//
//   conv_pix_mfma    out[co, m] = sum_R wt[R][co] * in[ci(R), pixel(m) shifted by tap(R)]
//       m runs over (output pixel, image) with pixels fastest -- the memory-contiguous axis of every tensor
//       here -- and sits on the MFMA "B / column" side, so each accumulator register of a lane is one
//       channel and 32 consecutive lanes are 32 consecutive pixels: stores are 128-byte runs.
//       Forward:        in = x,    R = (i,j,c), out = y,    tap shift = (i*dilate - pad) on a strided grid.
//       Backward-data:  in = dzdy, R = (i,j,k), out = dzdx, tap shift = (pad - i*dilate), stride 1.
//       The filter bank is first rewritten as wt[R][co] (co contiguous, zero padded to tile multiples) by a
//       small prologue kernel so weight tiles load as 16-byte vectors with no bounds tests.
//
//   conv_wgrad_mfma  dF[R, k] = sum_m xg[R, m] * dzdy[k, m],  xg = the (never materialised) patch matrix.
//       The reduction axis m (pixels x images) is split across workgroups; each writes a partial filter
//       bank and a second kernel adds the partials in a fixed order (deterministic, no atomics).
//       R sits on the MFMA column side, so stores run along the contiguous axis of dF.
//
// Work decomposition: 256 threads = 4 wavefronts; a wavefront owns WA x WB blocks of 32 x 32 accumulators;
// LDS tiles are double buffered with one barrier per reduction step; global loads for step i+1 are issued
// before the MFMAs of step i and parked in registers.
#include "conv_common.hpp"

#include <algorithm>
#include <atomic>

namespace mcn {
namespace {


constexpr int kMaxTaps = 128;

// ------------------------------------------------------------------------------------------------
// pixel-major kernel (forward / backward-data)
// ------------------------------------------------------------------------------------------------


// wt[R][co] from the MATLAB filter bank f[i,j,c,k] (FV x K, column-major), t = i + FH*j.
//   reduction row R = t + T*ci (channel-major) or, when tapMajor (Cin a multiple of 16), in chunks of 16 channels
//   with the taps inside a chunk: R = c16 + 16*(t + T*chunk), ci = 16*chunk + c16.  Walking the taps of a few
//   channels before moving to the next channels re-reads the same pixels (shifted by a tap) back to back, while
//   they are still in L1 / L2; tap-outermost order re-read the whole channel range between two visits, which sent
//   3x3 layers through the memory fabric 8 times over.
//   forward:        ci = c, co = k : f[t + T*c + FV*k]
//   backward-data:  ci = k, co = c : f[t + T*(c + C*k)]
// Only the taps of the TapSet take part; T = nI*nJ, t = a + nI*b.
__device__ __forceinline__ void pack_element(float* __restrict__ wt, const float* __restrict__ f, const TapSet& ts, int Cin,
                                             int Cout, int rPad, int coutPad, int backward, int tapMajor, size_t idx) {
  if (idx >= (size_t)rPad * coutPad) return;
  const int T = ts.nI * ts.nJ;
  const int r = (int)(idx / coutPad), co = (int)(idx - (size_t)r * coutPad);
  float v = 0.f;
  if (r < T * Cin && co < Cout) {
    int ci, t;
    if (tapMajor) {
      const int chunk = r / (16 * T), rem = r - chunk * 16 * T;
      t = rem / 16;
      ci = chunk * 16 + (rem - t * 16);
    } else {
      ci = r / T;
      t = r - ci * T;
    }
    const int b = t / ts.nI, a = t - b * ts.nI;
    const size_t Tf = (size_t)ts.FH * ts.FW;
    const size_t tf = (size_t)(ts.i0 + a * ts.iStep) + (size_t)ts.FH * (ts.j0 + b * ts.jStep);
    v = backward ? f[tf + Tf * (co + (size_t)Cout * ci)] : f[tf + Tf * ci + Tf * Cin * co];
  }
  wt[idx] = v;
}

// Forward banks with every tap: wt[r][k] = f[v + FV*k], v = t + T*c the position in the filter volume and r = v or its
// tap-major permutation.  Element by element (above) the lanes of a wavefront run along k and read f a whole filter
// volume apart.  Here a workgroup moves a tile of 64 volume positions x 64 filters through LDS: the reads run along the
// volume, the writes along the filters (all banks of ResNet-50 in one launch: 0.12 ms less per training step).
__device__ __forceinline__ void pack_tile(float* __restrict__ wt, const float* __restrict__ f, int T, int Cin, int Cout,
                                          int rPad, int coutPad, int tapMajor, unsigned tile, float (*lds)[65]) {
  const unsigned tilesK = (unsigned)(coutPad + 63) / 64;
  const int v0 = (int)(tile / tilesK) * 64, k0 = (int)(tile % tilesK) * 64;
  const int FV = T * Cin;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  // (all 16 loads of a thread in flight at once: a small bank is a handful of tiles, and its packing is one round trip)
  float got[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int k = k0 + w * 16 + i, v = v0 + lane;
    got[i] = (k < Cout && v < FV) ? f[(size_t)FV * k + v] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) lds[w * 16 + i][lane] = got[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int v = v0 + w * 16 + i;
    int r = v;
    if (tapMajor && v < FV) {
      const int ci = v / T, t = v - ci * T;
      r = (ci & 15) + 16 * (t + T * (ci >> 4));
    }
    if (v < rPad && k0 + lane < coutPad) wt[(size_t)r * coutPad + k0 + lane] = lds[lane][w * 16 + i];
  }
}

// (`tapMajor` carries two flags: 1 = tap-major rows, 2 = tile by tile)
__global__ __launch_bounds__(256) void conv_pack_weights(float* __restrict__ wt, const float* __restrict__ f,
                                                         TapSet ts, int Cin, int Cout, int rPad, int coutPad,
                                                         int backward, int tapMajor) {
  __shared__ float lds[64][65];
  if (tapMajor & 2) pack_tile(wt, f, ts.nI * ts.nJ, Cin, Cout, rPad, coutPad, tapMajor & 1, blockIdx.x, lds);
  else pack_element(wt, f, ts, Cin, Cout, rPad, coutPad, backward, tapMajor, (size_t)blockIdx.x * 256 + threadIdx.x);
}

// Many banks in one launch: workgroup b belongs to the job whose [firstBlock, firstBlock + blocks) holds b.
__global__ __launch_bounds__(256) void conv_pack_many(const PackJob* __restrict__ jobs, int nJobs) {
  __shared__ float lds[64][65];
  int lo = 0, hi = nJobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (jobs[mid].firstBlock <= blockIdx.x) lo = mid;
    else hi = mid - 1;
  }
  const PackJob j = jobs[lo];
  if (j.tapMajor & 2) pack_tile(j.wt, j.f, j.taps.nI * j.taps.nJ, j.Cin, j.Cout, j.rPad, j.coutPad, j.tapMajor & 1, blockIdx.x - j.firstBlock, lds);
  else pack_element(j.wt, j.f, j.taps, j.Cin, j.Cout, j.rPad, j.coutPad, j.backward, j.tapMajor,
                    (size_t)(blockIdx.x - j.firstBlock) * 256 + threadIdx.x);
}

// tile by tile: forward banks of all taps -- in a launch of their own only from 32 tiles on (a small bank is packed
// sooner by many workgroups of one element per thread than by a handful of tiles); the flags for `tapMajor`
int pack_flags(const TapSet& ts, int backward, bool tapMajor, int rPad, int coutPad, bool batched) {
  const bool tiled = !backward && ts.nI == ts.FH && ts.nJ == ts.FW && ts.i0 == 0 && ts.j0 == 0 && ts.iStep == 1 &&
                     ts.jStep == 1 && (batched || (long long)((rPad + 63) / 64) * ((coutPad + 63) / 64) >= 32);
  return (tapMajor ? 1 : 0) | (tiled ? 2 : 0);
}
unsigned pack_blocks(int flags, int rPad, int coutPad) {
  return (flags & 2) ? (unsigned)((rPad + 63) / 64) * (unsigned)((coutPad + 63) / 64)
                     : (unsigned)(((size_t)rPad * coutPad + 255) / 256);
}

// out = alpha * (sum of the partial results of a split reduction) + beta*out + bias.  The partials are dense tensors
// [n][co][q]; the destination is the layout the PixP describes (a dense tensor, one group's channels of a wider
// tensor, or one stride class of a backward-data product).  The partials are added in split order: deterministic.
// FLAT: the destination is the dense tensor itself (element i goes to element i) and n is a multiple of 4: 16-byte
// accesses, no index arithmetic beyond the bias channel.  Otherwise 32-bit indices with multiply-shift divisions
// (WIDE: tensors of 2^31 elements or more, plain 64-bit arithmetic).
template <bool FLAT, bool WIDE>
__global__ __launch_bounds__(256) void conv_pix_reduce(float* __restrict__ out, const float* __restrict__ partials,
                                                       const float* __restrict__ bias, size_t n, PixP p, FastDiv byCout) {
  if (FLAT) {
    const unsigned i4 = blockIdx.x * 256u + threadIdx.x;  // float4 index
    if ((size_t)i4 * 4 >= n) return;
    const v4f* src = (const v4f*)partials + i4;
    const size_t stride4 = (size_t)p.partStride / 4;
    v4f s = src[0];
    for (int k = 1; k < p.rSplits; ++k) s += src[(size_t)k * stride4];
    v4f v = p.alpha * s;
    if (p.beta != 0.f) {
      const v4f o = ((const v4f*)out)[i4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = fmaf(p.beta, o[j], v[j]);
    }
    if (bias) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int plane = p.byQ.div((int)(i4 * 4 + j));
        v[j] += bias[plane - byCout.div(plane) * p.Cout];
      }
    }
    ((v4f*)out)[i4] = v;
    return;
  }
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = partials[i];
  for (int k = 1; k < p.rSplits; ++k) s += partials[(size_t)k * p.partStride + i];
  int q, co;
  size_t img;
  if (WIDE) {
    const int Q = p.OH * p.OW;
    const size_t plane = i / Q;
    q = (int)(i - plane * Q);
    co = (int)(plane % p.Cout);
    img = plane / p.Cout;
  } else {
    int plane, im;
    p.byQ.divmod((int)i, &plane, &q);
    byCout.divmod(plane, &im, &co);
    img = (size_t)im;
  }
  float* dst = out + img * (size_t)p.outImg + (size_t)co * p.outPlane + out_pixel_offset(p, q);
  float v = p.alpha * s;
  if (p.beta != 0.f) v = fmaf(p.beta, *dst, v);
  if (bias) v += bias[co];
  *dst = v;
}

// UT ("uniform tap"): Cin is a multiple of 16 and the reduction runs in chunks of 16 channels, tap by tap inside
// a chunk (see conv_pack_weights), so all 16 rows of a step share one tap: the tap's shift and the inside-the-image test are computed once per step and
// thread, the step's base address is uniform (scalar registers), and every gathered row is a load at a
// per-thread constant 32-bit offset from it.  This removes almost all vector-ALU work from the loop, and
// vector-ALU work is what competes with the MFMAs for the SIMD.
// DIRECT (with UT; pixel tiles of at least 64, channel tiles of at least 64): the loads of a step go from global memory
// straight into LDS (buffer loads with the LDS destination), a few at a time between the MFMAs of the step in hand: no
// staging registers, no LDS write instructions.  Both tiles are laid out in LDS exactly as a wavefront's load delivers
// them: 64 consecutive pixels of a row, or 64 consecutive 16-byte vectors of the bank's rows.
// (the kernel's body: workgroup `block` of the `blocks` that share the product `p`)
template <int WA, int WB, int NWA, int NWB, bool UT, bool DIRECT>
__device__ __forceinline__ void pix_body(float* __restrict__ out, const float* __restrict__ in, const float* __restrict__ wt,
                                         const float* __restrict__ bias, const PixP& p, const unsigned block,
                                         const unsigned blocks) {
  static_assert(NWA * NWB == 4, "four wavefronts per workgroup");
  static_assert(!DIRECT || (UT && WB * 32 * NWB >= 64 && WA * 32 * NWA >= 64), "loads into LDS: uniform taps, tiles of 64 and more");
  constexpr int BA = WA * 32 * NWA;  // output channels per workgroup
  constexpr int BB = WB * 32 * NWB;  // pixels per workgroup
  constexpr int BK = 16;             // reduction rows per step
  constexpr int PIXG = 256 / BB;     // thread groups sharing the pixel tile rows
  constexpr int RPT = BK / PIXG;     // gathered rows per thread and step
  constexpr int A4 = BK * BA / 4;    // float4s in a weight tile
  constexpr int APT = (A4 + 255) / 256;

  // DIRECT: loads run two steps ahead (they need no registers to wait in): three buffers, in dynamic LDS (with static
  // arrays the compiler makes every LDS read wait for all loads in flight, whatever buffer they fill)
  constexpr int NBUF = DIRECT ? 3 : 2;
  extern __shared__ float smem[];
  __shared__ float AsStatic[DIRECT ? 1 : 2][DIRECT ? 4 : BK * BA];
  __shared__ float BsStatic[DIRECT ? 1 : 2][DIRECT ? 4 : BK * BB];
  float* const AsBase = DIRECT ? smem : &AsStatic[0][0];
  float* const BsBase = DIRECT ? smem + NBUF * BK * BA : &BsStatic[0][0];
  auto As = [&](int b) -> float* { return AsBase + b * (BK * BA); };
  auto Bs = [&](int b) -> float* { return BsBase + b * (BK * BB); };
  __shared__ int2 tapStatic[DIRECT ? 1 : kMaxTaps];
  int2* const tapTab = DIRECT ? (int2*)(smem + NBUF * BK * (BA + BB)) : tapStatic;  // .x = dh + IH*dw, .y = (dh & 0xffff) | (dw << 16)

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kh = lane >> 5;
  const int wa = wave / NWB, wb = wave - wa * NWB;

  const int tilesA = (p.Cout + BA - 1) / BA;
  int logical = xcd_contiguous_id(block, blocks);
  int split = 0;
  if (p.rSplits > 1) {  // (split-major: the workgroups of one split are neighbours)
    const int tiles = (int)blocks / p.rSplits;
    split = logical / tiles;
    logical -= split * tiles;
    out += (size_t)split * p.partStride;
  }
  const int mt = logical / tilesA;
  const int co0 = (logical - mt * tilesA) * BA;
  const int m0 = mt * BB;

  const int IHW = p.IH * p.IW;

  if (tid < p.T) {
    const int j = tid / p.FH, i = tid - j * p.FH;
    const int dh = p.dhBase + i * p.dhStep, dw = p.dwBase + j * p.dwStep;
    tapTab[tid] = make_int2(dh + p.IH * dw, (int)((unsigned)(dh & 0xffff) | ((unsigned)dw << 16)));
  }

  // ---- this thread's pixel (fixed for the whole kernel)
  const int mm = tid % BB, pg = tid / BB;
  const int m = m0 + mm;
  const bool mvalid = m < p.M;
  int ihB = 0, iwB = 0;
  const float* inN = in;
  {
    int n, q, ow, oh;
    p.byQ.divmod(mvalid ? m : 0, &n, &q);
    p.byOH.divmod(q, &ow, &oh);
    ihB = oh * p.sy;
    iwB = ow * p.sx;
    inN = in + (size_t)n * p.inImg + ihB + p.IH * iwB;
  }
  // first gathered row of this thread: R = pg*RPT -> (tap, channel); advanced by BK per step
  const int nStepsAll = (p.R + BK - 1) / BK;
  const int sBegin = split * p.stepsPerSplit;
  const int sEnd = p.rSplits > 1 ? min(nStepsAll, sBegin + p.stepsPerSplit) : nStepsAll;
  int ciS, tapS;
  p.byT.divmod(pg * RPT + sBegin * BK, &ciS, &tapS);
  const int advC = p.advC, advT = p.advT;
  // UT: per-thread constant element offsets (relative to `in`) of this thread's RPT channels at tap shift 0,
  // and the uniform (tap, first channel) of the step being fetched
  int offE[RPT];
  int utTap = 0, utCi = 0;  // step s of the chunked order: tap s % T of channels 16*(s / T) ...
  if (UT) {
    const int pix = (int)(inN - in);
#pragma unroll
    for (int e = 0; e < RPT; ++e) offE[e] = pix + (pg * RPT + e) * IHW;
  }

  floatx16 acc[WA][WB];
#pragma unroll
  for (int a = 0; a < WA; ++a)
#pragma unroll
    for (int b = 0; b < WB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  float pb[RPT];
  float4 pa0 = make_float4(0.f, 0.f, 0.f, 0.f), pa1 = pa0;  // parked weight vectors (APT <= 2)
  static_assert(APT <= 2, "at most two weight vectors per thread and step");
  unsigned okMask = 0;  // bit e: gathered row e of the parked step lies inside the image
  if (UT && sBegin > 0) {
    const int chunk = p.byT.div(sBegin);
    utTap = sBegin - chunk * p.T;
    utCi = chunk * BK;
  }

  // Issues the global loads of one step and parks them in registers.  Straight-line on purpose: the tap
  // table reads go out together, and rows that fall outside the image load a dummy (the tensor's first
  // element) instead of branching, so all loads are in flight before anything waits; the mask zeroes them
  // when they are written to LDS.
  auto fetch = [&](int step) {
    if (UT) {
      const int2 tp = tapTab[utTap];
      const int shift = __builtin_amdgcn_readfirstlane(tp.x), packed = __builtin_amdgcn_readfirstlane(tp.y);
      const int ih = ihB + (int)(short)(packed & 0xffff), iw = iwB + (packed >> 16);
      const bool ok = mvalid && (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
      const float* base = in + (utCi * IHW + shift);  // uniform
      if (ok) {
#pragma unroll
        for (int e = 0; e < RPT; ++e) pb[e] = base[offE[e]];
      } else {
#pragma unroll
        for (int e = 0; e < RPT; ++e) pb[e] = 0.f;
      }
      if (++utTap == p.T) {  // the taps of these 16 channels, then the next 16 channels
        utTap = 0;
        utCi += BK;
      }
    } else {
      int2 tp[RPT];
      int cix[RPT];
      int t = tapS, ci = ciS;
#pragma unroll
      for (int e = 0; e < RPT; ++e) {
        tp[e] = tapTab[t];
        cix[e] = ci;
        if (++t == p.T) {
          t = 0;
          ++ci;
        }
      }
      okMask = 0;
#pragma unroll
      for (int e = 0; e < RPT; ++e) {
        const int ih = ihB + (int)(short)(tp[e].y & 0xffff);
        const int iw = iwB + (tp[e].y >> 16);
        const bool ok = mvalid && cix[e] < p.Cin && (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
        const float* src = ok ? inN + (cix[e] * IHW + tp[e].x) : in;
        pb[e] = *src;
        okMask |= ok ? (1u << e) : 0u;
      }
      ciS += advC;
      tapS += advT;
      if (tapS >= p.T) {
        tapS -= p.T;
        ++ciS;
      }
    }
    const float* wrow = wt + (size_t)step * BK * p.coutPad + co0;
    if (A4 % 256 == 0 || tid < A4) {
      const int row = tid / (BA / 4), c4 = tid - row * (BA / 4);
      pa0 = *(const float4*)(wrow + (size_t)row * p.coutPad + c4 * 4);
    }
    if (APT == 2) {
      const int idx = tid + 256;
      const int row = idx / (BA / 4), c4 = idx - row * (BA / 4);
      pa1 = *(const float4*)(wrow + (size_t)row * p.coutPad + c4 * 4);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int e = 0; e < RPT; ++e) Bs(buf)[(pg * RPT + e) * BB + mm] = (UT || ((okMask >> e) & 1u)) ? pb[e] : 0.f;
    if (A4 % 256 == 0 || tid < A4) *(float4*)&As(buf)[tid * 4] = pa0;
    if (APT == 2) *(float4*)&As(buf)[(tid + 256) * 4] = pa1;
  };
  // DIRECT: prep(step, live, buffer) works out the step's offsets (nothing is fetched when !live: the instruction stream
  // stays the same on the last step); issue(t) is load t of the step: the thread group's RPT gathered rows, then the
  // APT vectors of the bank.
  constexpr int NLOADS = RPT + APT;
  const int waveU = __builtin_amdgcn_readfirstlane(wave);
  __amdgpu_buffer_rsrc_t inr, wtr;
  unsigned voB = kOutside, voB0 = kOutside, voA[APT];
  int sB = 0, sA = 0;
  float *Bd = Bs(0), *Ad = As(0);
  if (DIRECT) {
    inr = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, (int)p.inBytes, 0x00020000);
    wtr = __builtin_amdgcn_make_buffer_rsrc((void*)wt, 0, (int)p.wtBytes, 0x00020000);
    // this lane's pixel, row 0 of its thread group, at tap shift 0
    voB0 = mvalid ? (unsigned)((int)(inN - in) + pg * RPT * IHW) * 4u : kOutside;
#pragma unroll
    for (int j = 0; j < APT; ++j) {
      const int idx = tid + 256 * j;
      const int row = idx / (BA / 4), c4 = idx - row * (BA / 4);
      voA[j] = (unsigned)(row * p.coutPad + c4 * 4) * 4u;
    }
  }
  // (the tap's shift as scalars kept up to date by additions, not from the table in LDS: the compiler makes a table
  // read wait for every load into LDS still in flight)
  int tapRow = utTap % p.FH, dhL = p.dhBase + tapRow * p.dhStep, dwL = p.dwBase + (utTap / p.FH) * p.dwStep;
  auto prep = [&](int step, bool live, int buf) {
    const int ih = ihB + dhL, iw = iwB + dwL;
    const bool ok = live && mvalid && (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
    voB = ok ? voB0 + (unsigned)((dhL + p.IH * dwL) * 4) : kOutside;  // (the shift may be negative: it goes with the lane's offset)
    sB = utCi * IHW * 4;
    dhL += p.dhStep;
    if (++tapRow == p.FH) {
      tapRow = 0;
      dhL = p.dhBase;
      dwL += p.dwStep;
    }
    if (++utTap == p.T) {
      utTap = 0;
      dwL = p.dwBase;
      utCi += BK;
    }
    sA = live ? (step * BK * p.coutPad + co0) * 4 : (int)kOutside;
    Bd = Bs(buf);
    Ad = As(buf);
  };
  auto issue = [&](int t) {
    typedef __attribute__((address_space(3))) void* lds_ptr;
    if (t < RPT) {  // gathered row pg RPT + t: this wavefront's 64 pixels of it
      const int pgU = (waveU * 64) / BB, mm0 = (waveU * 64) % BB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(inr, (lds_ptr)(Bd + (pgU * RPT + t) * BB + mm0), 4, (int)voB, sB + t * IHW * 4, 0, 0);
    } else {        // vectors 256 j + tid of the bank's 16 rows
      const int j = t - RPT;
      if (A4 % 256 == 0 || (256 * j + waveU * 64) < A4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(wtr, (lds_ptr)(Ad + (256 * j + waveU * 64) * 4), 16, (int)voA[j], sA, 0, 0);
    }
  };

  __syncthreads();  // tapTab ready
  if (DIRECT) {
    // two steps in flight before the loop (every wavefront issues NLOADS loads per step whether they fetch anything or
    // not, so "all but the youngest NLOADS have landed" is a count the hardware can wait for)
    prep(sBegin, sBegin < sEnd, 0);
#pragma unroll
    for (int t = 0; t < NLOADS; ++t) issue(t);
    prep(sBegin + 1, sBegin + 1 < sEnd, 1);
#pragma unroll
    for (int t = 0; t < NLOADS; ++t) issue(t);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(NLOADS) : "memory");
  } else {
    if (sBegin < sEnd) {
      fetch(sBegin);
      stash(0);
    }
    __syncthreads();
  }

  int buf = 0;  // (DIRECT: of three)
  for (int step = sBegin; step < sEnd; ++step) {
    if (!DIRECT) buf = (step - sBegin) & 1;
    if (DIRECT) prep(step + 2, step + 2 < sEnd, buf >= 1 ? buf - 1 : 2);  // = (buf + 2) % 3
    else if (step + 1 < sEnd) fetch(step + 1);
    const float* Ab = As(buf) + wa * WA * 32 + l32 + kh * BA;
    const float* Bb = Bs(buf) + wb * WB * 32 + l32 + kh * BB;
    // operand fragments are read one reduction pair ahead of the MFMAs that consume them
    float a[2][WA], b[2][WB];
#pragma unroll
    for (int ii = 0; ii < WA; ++ii) a[0][ii] = Ab[ii * 32];
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) b[0][jj] = Bb[jj * 32];
#pragma unroll
    for (int s = 0; s < BK / 2; ++s) {
      const int cur = s & 1, nxt = cur ^ 1;
      if (DIRECT) {
#pragma unroll
        for (int t = s * NLOADS / (BK / 2); t < (s + 1) * NLOADS / (BK / 2); ++t) issue(t);
      }
      if (s + 1 < BK / 2) {
#pragma unroll
        for (int ii = 0; ii < WA; ++ii) a[nxt][ii] = Ab[(2 * s + 2) * BA + ii * 32];
#pragma unroll
        for (int jj = 0; jj < WB; ++jj) b[nxt][jj] = Bb[(2 * s + 2) * BB + jj * 32];
      }
      __builtin_amdgcn_sched_barrier(0);  // keep the look-ahead reads ahead of this pair's MFMAs
#pragma unroll
      for (int ii = 0; ii < WA; ++ii)
#pragma unroll
        for (int jj = 0; jj < WB; ++jj)
          acc[ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][ii], b[cur][jj], acc[ii][jj], 0, 0, 0);
    }
    if (DIRECT) {
      // the next step's loads (issued a step ago) have landed; this step's own may still be in flight
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(NLOADS) : "memory");
      buf = buf == 2 ? 0 : buf + 1;
    } else {
      if (step + 1 < sEnd) stash(buf ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue: lane = pixel, register = channel
  const int waU = __builtin_amdgcn_readfirstlane(wa);  // a wavefront's tile position is uniform
  const int coW = co0 + waU * WA * 32;
  if (p.outBytes != 0 && coW + WA * 32 <= p.Cout) {
    // whole channel blocks inside the tensor: straight-line stores through a buffer descriptor
    const bufrsrc rsrc = make_bufrsrc(out, p.outBytes);
    const int plane = p.outPlane * 4;
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) {
      const int mo = m0 + wb * WB * 32 + jj * 32 + l32;
      int n, q;
      p.byQ.divmod(mo < p.M ? mo : 0, &n, &q);
      const unsigned vo = mo < p.M ? (unsigned)(n * p.outImg + out_pixel_offset(p, q) + 4 * kh * p.outPlane) * 4u : kOutside;
#pragma unroll
      for (int ii = 0; ii < WA; ++ii)
        store_block(acc[ii][jj], rsrc, vo, (coW + ii * 32) * plane, plane, p.alpha, p.beta,
                    bias ? bias + coW + ii * 32 : nullptr, kh);
    }
    return;
  }
#pragma unroll
  for (int jj = 0; jj < WB; ++jj) {
    const int mo = m0 + wb * WB * 32 + jj * 32 + l32;
    if (mo >= p.M) continue;
    int n, q;
    p.byQ.divmod(mo, &n, &q);
    float* o = out + (size_t)n * p.outImg + out_pixel_offset(p, q);
#pragma unroll
    for (int ii = 0; ii < WA; ++ii)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = co0 + wa * WA * 32 + ii * 32 + 8 * (r / 4) + 4 * kh + (r % 4);
        if (co < p.Cout) {
          float v = p.alpha * acc[ii][jj][r];
          if (p.beta != 0.f) v = fmaf(p.beta, o[(size_t)co * p.outPlane], v);
          if (bias) v += bias[co];
          o[(size_t)co * p.outPlane] = v;
        }
      }
  }
}

template <int WA, int WB, int NWA, int NWB, bool UT, bool DIRECT = false>
__global__ __launch_bounds__(256, 2) void conv_pix_mfma(float* __restrict__ out, const float* __restrict__ in,
                                                        const float* __restrict__ wt,
                                                        const float* __restrict__ bias, PixP p) {
  pix_body<WA, WB, NWA, NWB, UT, DIRECT>(out, in, wt, bias, p, blockIdx.x, gridDim.x);
}

// Up to four products over the same two tensors in one launch (the stride classes of a strided layer's backward-data
// product: each a small product of its own, with its own taps, bank and sub-grid of the output).  Workgroups
// [first[i], first[i + 1]) belong to product i; the longest reductions come first.  Always the form with uniform taps
// and loads straight into LDS.
constexpr int kMaxMulti = 4;
struct PixMulti {
  PixP p[kMaxMulti];
  const float* wt[kMaxMulti];
  unsigned first[kMaxMulti + 1];
  int n;
};

template <int WA, int WB, int NWA, int NWB>
__global__ __launch_bounds__(256, 2) void conv_pix_multi(float* __restrict__ out, const float* __restrict__ in, PixMulti m) {
  int i = 0;
#pragma unroll
  for (int j = 1; j < kMaxMulti; ++j)
    if (j < m.n && blockIdx.x >= m.first[j]) i = j;
  pix_body<WA, WB, NWA, NWB, true, true>(out, in, m.wt[i], nullptr, m.p[i], blockIdx.x - m.first[i], m.first[i + 1] - m.first[i]);
}

// ------------------------------------------------------------------------------------------------
// filter-gradient kernel
// ------------------------------------------------------------------------------------------------

struct WgP {
  int H, W, C, K;
  int OH, OW;
  int FH, T;
  int sy, sx, pt, pl, dly, dlx;
  int FV;
  int M;                 // OH*OW*N (< 2^31)
  int chunkSpan;         // pixels per split (multiple of 32)
  int splits;
  FastDiv byQ, byOH, byT, byFH, byTiles, byTilesK, byC;
  unsigned outBytes;     // size of the partial banks, or 0 when they do not fit a 2 GiB buffer descriptor
  int xImg, dyImg;       // elements between images of x and of dzdy (wider than C*H*W, K*OH*OW for a filter group)
  unsigned xBytes, dyBytes;  // bytes from x / dzdy to the end of what this product reads (UT: both < 2 GiB)
};

// UT ("uniform tap"): rows are ordered tap-major (R' = c + C*t) and C is a multiple of 32, so each 32-row MFMA
// block lies inside one tap.  A thread's sixteen patch rows then need four inside-the-image tests per step
// instead of sixteen, and every load is a per-thread constant 32-bit offset from a per-step pixel offset.
// The partial banks come out in R' order; conv_wgrad_reduce puts them back in MATLAB order.
// DIRECT (with UT, all filter rows of every tile present): the loads of a step go from global memory straight into LDS
// (buffer loads with the LDS destination: no staging registers, no LDS write instructions, nothing to wait for
// before the next step's MFMAs but the barrier).  A wavefront's load instruction fills 64 consecutive floats of LDS,
// so a pair of rows (the two halves of the wavefront) lies side by side and pairs are 65 floats apart: row r, pixel p
// at (r / 2) 65 + (r % 2) 32 + p -- the 32 rows a fragment read touches fall into 32 different banks.
// (LDS buffers of the filter-gradient kernel.  DEEP: three also for larger tiles -- one workgroup to a CU then, so only
// for launches that have no more workgroups than CUs anyway)
constexpr int wgrad_buffers(int BA, int BB, bool direct, bool deep) { return direct && (BA + BB <= 192 || deep) ? 3 : 2; }

template <int WA, int WB, int NWA, int NWB, bool UT, bool DIRECT = false, bool DEEP = false>
__global__ __launch_bounds__(256, 2) void conv_wgrad_mfma(float* __restrict__ out, const float* __restrict__ x,
                                                          const float* __restrict__ dy, WgP p) {
  static_assert(NWA * NWB == 4, "four wavefronts per workgroup");
  static_assert(!DIRECT || UT, "loads into LDS go with the uniform-tap row order");
  constexpr int BA = WA * 32 * NWA;  // filters (k) per workgroup
  constexpr int BB = WB * 32 * NWB;  // filter-volume rows (R) per workgroup
  constexpr int BP = 32;             // pixels per reduction step
  constexpr int LD = BP + 1;         // padded LDS pitch: column reads hit 32 distinct banks
  constexpr int APT = BA / 8, BPT = BB / 8;

  // dynamic LDS (the 128 x 128 configuration needs 67 KB, above the 64 KB static limit).  DIRECT tiles of up to 192
  // rows take three buffers (two workgroups still fit a CU): their loads run two steps ahead, and the barrier at the
  // end of a step waits only for the step before them
  constexpr int NBUF = wgrad_buffers(BA, BB, DIRECT, DEEP);
  extern __shared__ float smem[];
  float(*As)[BA * LD] = (float(*)[BA * LD])smem;                     // [NBUF][BA*LD]
  float(*Bs)[BB * LD] = (float(*)[BB * LD])(smem + NBUF * BA * LD);  // [NBUF][BB*LD]
  int2* rowTab = (int2*)(smem + NBUF * (BA + BB) * LD);              // [BB] .x = c*H*W + dh + H*dw, .y = dh | dw << 16

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kh = lane >> 5;
  const int wa = wave / NWB, wb = wave - wa * NWB;

  const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
  int split, tile, rt, kt;
  p.byTiles.divmod(logical, &split, &tile);
  p.byTilesK.divmod(tile, &rt, &kt);
  const int k0 = kt * BA;
  const int r0 = rt * BB;

  const int HW = p.H * p.W;
  const int Q = p.OH * p.OW;

  if (!UT && tid < BB) {
    const int R = r0 + tid;
    int2 e = make_int2(0, 0x8000);  // dh = -32768: never inside the image
    if (R < p.FV) {
      int c, t, j, i;
      p.byT.divmod(R, &c, &t);
      p.byFH.divmod(t, &j, &i);
      const int dh = i * p.dly - p.pt, dw = j * p.dlx - p.pl;
      e = make_int2(c * HW + dh + p.H * dw, (int)((unsigned)(dh & 0xffff) | ((unsigned)dw << 16)));
    }
    rowTab[tid] = e;
  }

  const int mBegin = split * p.chunkSpan;
  const int mEnd = min(mBegin + p.chunkSpan, p.M);
  const int nSteps = mEnd > mBegin ? (mEnd - mBegin + BP - 1) / BP : 0;

  const int px = tid & 31, rg = tid >> 5;

  floatx16 acc[WA][WB];
#pragma unroll
  for (int a = 0; a < WA; ++a)
#pragma unroll
    for (int b = 0; b < WB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  float pa[APT], pb[BPT];
  unsigned okA = 0, okB = 0;

  // UT: per 32-row block its tap shift (uniform).  The loads are buffer loads: the per-lane offset is the pixel (plus one
  // row for the upper half of the wavefront: thread group rg = 2 wave + half), the scalar offset is the row -- no
  // address arithmetic per load in vector registers, and a pixel outside the image or past the split's end uses an
  // offset beyond the tensor, for which the hardware returns 0 (no branches, no dummy reads).
  constexpr int NBLK = BB / 32;
  int blkDh[NBLK], blkDw[NBLK], blkShift[NBLK];
  int xOffS[BPT], yOffS[APT];  // byte offsets of this wavefront's rows at half 0 (uniform: scalar registers)
  unsigned kPresent = 0;
  const int waveU = __builtin_amdgcn_readfirstlane(wave);
  const int half = rg & 1;
  __amdgpu_buffer_rsrc_t xr, yr;
  if (UT) {
    xr = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)p.xBytes, 0x00020000);
    yr = __builtin_amdgcn_make_buffer_rsrc((void*)dy, 0, (int)p.dyBytes, 0x00020000);
#pragma unroll
    for (int jb = 0; jb < NBLK; ++jb) {
      const int Rb = r0 + 32 * jb;
      int t, cb, j, i;
      p.byC.divmod(Rb < p.FV ? Rb : 0, &t, &cb);
      p.byFH.divmod(t, &j, &i);
      const int dh = i * p.dly - p.pt, dw = j * p.dlx - p.pl;
      blkDh[jb] = Rb < p.FV ? dh : -32768;  // absent block: never inside the image
      blkDw[jb] = dw;
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) xOffS[4 * jb + e4] = (cb + 2 * waveU + 8 * e4) * HW * 4;
      blkShift[jb] = (dh + p.H * dw) * 4;  // (added to the lane's offset, and only where the shifted pixel is inside the image)
    }
#pragma unroll
    for (int e = 0; e < APT; ++e) {
      const int kE = k0 + 2 * waveU + 8 * e;  // (row of half 0; half 1 reads the row after it)
      yOffS[e] = (kE < p.K ? kE : 0) * Q * 4;
      kPresent |= kE + half < p.K ? (1u << e) : 0u;
    }
  }

  // Straight-line like the pixel-major kernel's: table reads first, then every load (absent elements read a
  // dummy and are zeroed by mask when written to LDS).
  auto fetch = [&](int step) {
    const int m = mBegin + step * BP + px;
    const bool valid = m < mEnd;
    int n, q, ow, oh;
    p.byQ.divmod(valid ? m : mBegin, &n, &q);
    p.byOH.divmod(q, &ow, &oh);
    const int ihB = oh * p.sy, iwB = ow * p.sx;
    if (UT) {
      const unsigned pixX = (unsigned)(n * p.xImg + ihB + p.H * iwB + half * HW) * 4u;
      const unsigned pixY = valid ? (unsigned)(n * p.dyImg + q + half * Q) * 4u : kOutside;
#pragma unroll
      for (int jb = 0; jb < NBLK; ++jb) {
        const bool ok = valid && (unsigned)(ihB + blkDh[jb]) < (unsigned)p.H && (unsigned)(iwB + blkDw[jb]) < (unsigned)p.W;
        const unsigned vo = ok ? pixX + (unsigned)blkShift[jb] : kOutside;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
          pb[4 * jb + e4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, (int)vo, xOffS[4 * jb + e4], 0));
      }
#pragma unroll
      for (int e = 0; e < APT; ++e)
        pa[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, (int)pixY, yOffS[e], 0));
      okA = kPresent;
      okB = 0xffffffffu;
      return;
    }
    const float* xN = x + (size_t)n * p.xImg + ihB + p.H * iwB;
    const float* dyN = dy + (size_t)n * p.dyImg + q;
    int2 tp[BPT];
#pragma unroll
    for (int e = 0; e < BPT; ++e) tp[e] = rowTab[rg + 8 * e];
    okB = 0;
#pragma unroll
    for (int e = 0; e < BPT; ++e) {
      const int ih = ihB + (int)(short)(tp[e].y & 0xffff);
      const int iw = iwB + (tp[e].y >> 16);
      const bool ok = valid && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
      const float* src = ok ? xN + tp[e].x : x;
      pb[e] = *src;
      okB |= ok ? (1u << e) : 0u;
    }
    okA = 0;
#pragma unroll
    for (int e = 0; e < APT; ++e) {
      const int k = k0 + rg + 8 * e;
      const bool ok = valid && k < p.K;
      const float* src = ok ? dyN + (size_t)k * Q : dy;
      pa[e] = *src;
      okA |= ok ? (1u << e) : 0u;
    }
  };
  // DIRECT: the loads of the next step are issued a few at a time between the MFMAs of the step in hand (all at once at
  // the top of a step they hold up that wavefront's first MFMAs).  prep: the per-lane offsets of step `step` (nothing
  // is fetched when !live: the instruction stream stays the same on the last step); issue(t): load t of the step.
  constexpr int NLOADS = BPT + APT;
  constexpr int SPREAD = BP / 2;  // pairs of a step the loads are spread over (over the first 8 or 12 only: same times)
  unsigned voX[NBLK], voY = kOutside;
  float *Bd = Bs[0], *Ad = As[0];
  int bufL = 0;  // the buffer the next prepared step loads into (steps take the buffers in turn)
  auto prep = [&](int step, bool live) {
    const int m = mBegin + step * BP + px;
    const bool valid = live && m < mEnd;
    int n, q, ow, oh;
    p.byQ.divmod(valid ? m : mBegin, &n, &q);
    p.byOH.divmod(q, &ow, &oh);
    const int ihB = oh * p.sy, iwB = ow * p.sx;
    const unsigned pixX = (unsigned)(n * p.xImg + ihB + p.H * iwB + half * HW) * 4u;
#pragma unroll
    for (int jb = 0; jb < NBLK; ++jb) {
      const bool ok = valid && (unsigned)(ihB + blkDh[jb]) < (unsigned)p.H && (unsigned)(iwB + blkDw[jb]) < (unsigned)p.W;
      voX[jb] = ok ? pixX + (unsigned)blkShift[jb] : kOutside;
    }
    voY = valid ? (unsigned)(n * p.dyImg + q + half * Q) * 4u : kOutside;
    Bd = Bs[bufL];
    Ad = As[bufL];
    bufL = bufL == NBUF - 1 ? 0 : bufL + 1;
  };
  auto issue = [&](int t) {
    typedef __attribute__((address_space(3))) void* lds_ptr;
    if (t < BPT) {  // x: rows 32 jb + 2 wave + 8 e4 (+ half) = pair 16 jb + wave + 4 e4
      const int jb = t / 4, e4 = t % 4;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (lds_ptr)(Bd + (16 * jb + waveU + 4 * e4) * 65), 4, (int)voX[jb], xOffS[t], 0, 0);
    } else {        // dzdy: rows 2 wave + 8 e (+ half) = pair wave + 4 e
      const int e = t - BPT;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(yr, (lds_ptr)(Ad + (waveU + 4 * e) * 65), 4, (int)voY, yOffS[e], 0, 0);
    }
  };
  const bool allK = k0 + BA <= p.K;  // uniform: no filter row of this tile is absent
  auto stash = [&](int buf) {
#pragma unroll
    for (int e = 0; e < BPT; ++e) Bs[buf][(rg + 8 * e) * LD + px] = (UT || ((okB >> e) & 1u)) ? pb[e] : 0.f;
    if (UT && allK) {
#pragma unroll
      for (int e = 0; e < APT; ++e) As[buf][(rg + 8 * e) * LD + px] = pa[e];
    } else {
#pragma unroll
      for (int e = 0; e < APT; ++e) As[buf][(rg + 8 * e) * LD + px] = ((okA >> e) & 1u) ? pa[e] : 0.f;
    }
  };

  __syncthreads();  // rowTab ready
  if (nSteps > 0) {
    if (DIRECT) {
      prep(0, true);
#pragma unroll
      for (int t = 0; t < NLOADS; ++t) issue(t);
      if (NBUF == 3) {
        prep(1, 1 < nSteps);
#pragma unroll
        for (int t = 0; t < NLOADS; ++t) issue(t);
      }
    } else {
      fetch(0);
      stash(0);
    }
  }
  // (this wavefront's loads into LDS for the first step have landed; with three buffers the second step's stay in flight:
  // every wavefront issues NLOADS loads per step whether they fetch anything or not, so the count is exact)
  if (DIRECT && NBUF == 3) {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(NLOADS) : "memory");
  } else {
    if (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  // floats between the rows of consecutive 32-row blocks, and this lane's row inside its first block
  constexpr int BLK = DIRECT ? 16 * 65 : 32 * LD;
  const int laneRow = DIRECT ? (l32 >> 1) * 65 + (l32 & 1) * 32 : l32 * LD;
  int buf = 0;
  for (int step = 0; step < nSteps; ++step) {
    if (DIRECT) prep(step + NBUF - 1, step + NBUF - 1 < nSteps);
    else if (step + 1 < nSteps) fetch(step + 1);
    const float* Ab = As[buf] + wa * WA * BLK + laneRow + kh;
    const float* Bb = Bs[buf] + wb * WB * BLK + laneRow + kh;
    float a[2][WA], b[2][WB];
#pragma unroll
    for (int ii = 0; ii < WA; ++ii) a[0][ii] = Ab[ii * BLK];
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) b[0][jj] = Bb[jj * BLK];
#pragma unroll
    for (int s = 0; s < BP / 2; ++s) {
      const int cur = s & 1, nxt = cur ^ 1;
      if (DIRECT && s < SPREAD) {
#pragma unroll
        for (int t = s * NLOADS / SPREAD; t < (s + 1) * NLOADS / SPREAD; ++t) issue(t);
      }
      if (s + 1 < BP / 2) {
#pragma unroll
        for (int ii = 0; ii < WA; ++ii) a[nxt][ii] = Ab[ii * BLK + 2 * s + 2];
#pragma unroll
        for (int jj = 0; jj < WB; ++jj) b[nxt][jj] = Bb[jj * BLK + 2 * s + 2];
      }
      __builtin_amdgcn_sched_barrier(0);  // keep the look-ahead reads ahead of this pair's MFMAs
#pragma unroll
      for (int ii = 0; ii < WA; ++ii)
#pragma unroll
        for (int jj = 0; jj < WB; ++jj)
          acc[ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][ii], b[cur][jj], acc[ii][jj], 0, 0, 0);
    }
    if (!DIRECT && step + 1 < nSteps) stash(buf ^ 1);
    if (DIRECT && NBUF == 3) {
      // the next step's loads (issued a step ago) have landed; this step's own may still be in flight
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::"n"(NLOADS) : "memory");
    } else {
      if (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    buf = buf == NBUF - 1 ? 0 : buf + 1;
  }

  // ---- epilogue: lane = filter-volume row R (contiguous in dF), register = filter k
  const int waU = __builtin_amdgcn_readfirstlane(wa);  // a wavefront's tile position is uniform
  const int kW = k0 + waU * WA * 32;
  if (p.outBytes != 0 && kW + WA * 32 <= p.K) {
    // whole filter blocks present: straight-line stores through a buffer descriptor
    const bufrsrc rsrc = make_bufrsrc(out, p.outBytes);
    const int plane = p.FV * 4;
    const int sbase = __builtin_amdgcn_readfirstlane(split) * p.K * plane;
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) {
      const int R = r0 + wb * WB * 32 + jj * 32 + l32;
      const unsigned vo = R < p.FV ? (unsigned)(R + 4 * kh * p.FV) * 4u : kOutside;
#pragma unroll
      for (int ii = 0; ii < WA; ++ii)
        store_block(acc[ii][jj], rsrc, vo, sbase + (kW + ii * 32) * plane, plane, 1.f, 0.f, nullptr, kh);
    }
    return;
  }
  float* o = out + (size_t)split * p.FV * p.K;
#pragma unroll
  for (int jj = 0; jj < WB; ++jj) {
    const int R = r0 + wb * WB * 32 + jj * 32 + l32;
    if (R >= p.FV) continue;
#pragma unroll
    for (int ii = 0; ii < WA; ++ii)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int k = k0 + wa * WA * 32 + ii * 32 + 8 * (r / 4) + 4 * kh + (r % 4);
        if (k < p.K) o[(size_t)R + (size_t)p.FV * k] = acc[ii][jj][r];
      }
  }
}

// dF[e] = sum over splits.  A workgroup owns 64 consecutive elements; thread (e, g) adds the splits
// g, g+4, g+8, ... (four independent load streams per element, each unrolled eight deep: 256 and 512 splits of the
// 56x56 layers 9.9 -> 8.0 us), then the four partial sums are combined through LDS in a fixed order.  Deterministic.
__device__ __forceinline__ void wgrad_reduce_block(float* __restrict__ df, const float* __restrict__ partials, size_t n,
                                                   int splits, int tapMajor, int C, int T, unsigned block, float (*part)[64]) {
  const int e = threadIdx.x & 63, g = threadIdx.x >> 6;
  const size_t i = (size_t)block * 64 + e;
  float s = 0.f;
  if (i < n) {
    int k = g;
    // (eight loads in flight per thread, then four: a wavefront waits for all its loads before it adds)
#pragma unroll 1
    for (; k + 28 < splits; k += 32) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partials[(size_t)(k + 4 * u) * n + i];
      s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
#pragma unroll 1
    for (; k + 12 < splits; k += 16) {
      const float a = partials[(size_t)k * n + i], b = partials[(size_t)(k + 4) * n + i];
      const float c = partials[(size_t)(k + 8) * n + i], d = partials[(size_t)(k + 12) * n + i];
      s += (a + b) + (c + d);
    }
    for (; k < splits; k += 4) s += partials[(size_t)k * n + i];
  }
  part[g][e] = s;
  __syncthreads();
  if (g == 0 && i < n) {
    size_t o = i;
    if (tapMajor) {  // partial banks are indexed c + C*t + FV*k; MATLAB order is t + T*c + FV*k
      const size_t FV = (size_t)C * T;
      const size_t k = i / FV, r = i - k * FV;
      const size_t t = r / C, c = r - t * C;
      o = t + (size_t)T * c + FV * k;
    }
    df[o] = (part[0][e] + part[1][e]) + (part[2][e] + part[3][e]);
  }
}

__global__ __launch_bounds__(256) void conv_wgrad_reduce(float* __restrict__ df, const float* __restrict__ partials,
                                                         size_t n, int splits, int tapMajor, int C, int T) {
  __shared__ float part[4][64];
  wgrad_reduce_block(df, partials, n, splits, tapMajor, C, T, blockIdx.x, part);
}

// The sums of many filter gradients in one launch: workgroup b belongs to the job whose [firstBlock, firstBlock +
// blocks) holds b.
__global__ __launch_bounds__(256) void conv_wgrad_reduce_many(const ReduceJob* __restrict__ jobs, int nJobs) {
  __shared__ float part[4][64];
  int lo = 0, hi = nJobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (jobs[mid].firstBlock <= blockIdx.x) lo = mid;
    else hi = mid - 1;
  }
  const ReduceJob j = jobs[lo];
  wgrad_reduce_block(j.df, j.partials, j.n, j.splits, j.tapMajor, j.C, j.T, blockIdx.x - j.firstBlock, part);
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------

int pick_channels_tile(int cout) { return cout > 64 ? 128 : (cout > 32 ? 64 : 32); }

bool common_ok(const ConvP& p) {
  // tap offsets are packed as 16-bit fields and "row absent" is encoded as offset -32768
  const long long spanH = (long long)p.H + p.pt + (long long)p.FH * p.dy, spanW = (long long)p.W + p.pl + (long long)p.FW * p.dx;
  return p.FH * p.FW <= kMaxTaps && spanH < 32768 && spanW < 32768 &&
         (long long)p.outH * p.outW * p.N < (1ll << 31) && (long long)p.H * p.W * p.N < (1ll << 31) &&
         (long long)p.H * p.W * p.C < (1ll << 31) && (long long)p.outH * p.outW * p.K < (1ll << 31);
}

// One filter group of a layer as a layer of its own: FC input channels, K/groups filters.  Its tensors are slices
// of the layer's (the image strides stay those of the whole layer: struct Wide).
ConvP group_view(const ConvP& p) {
  ConvP g = p;
  g.C = p.FC;
  g.K = p.Kg;
  g.groups = 1;
  return g;
}

// A layer whose filters cover its whole (unpadded) input makes one output pixel per image: a fully-connected
// layer.  In memory x is then the matrix (H*W*C) x N and the bank (H*W*C) x K, which is exactly a 1x1 layer over a
// 1x1 image with H*W*C channels -- the reference's special case too (bits/nnfullyconnected.cu:30-185: plain GEMMs).
// Seen that way the reduction has one tap and H*W*C rows instead of H*W taps of which each output pixel of the
// backward-data product uses one.
ConvP fc_view(const ConvP& p) {
  if (!(p.groups == 1 && p.FH == p.H && p.FW == p.W && p.pt == 0 && p.pl == 0 && p.outH == 1 && p.outW == 1 &&
        p.dy == 1 && p.dx == 1) || (p.H == 1 && p.W == 1) || (long long)p.H * p.W * p.C >= (1ll << 31))
    return p;
  ConvP v = p;
  v.C = v.FC = p.H * p.W * p.C;
  v.H = v.W = v.FH = v.FW = 1;
  v.sy = v.sx = 1;
  return v;
}

struct Wide {
  int xImg, yImg;  // elements between images of the layer's input and output tensors
};

Wide wide_of(const ConvP& p) { return Wide{p.C * p.H * p.W, p.K * p.outH * p.outW}; }

// the tap-major variant of the filter-gradient kernel: 32-row blocks inside one tap, 32-bit element offsets
// (takes the whole layer, not a group view: the offsets span the whole tensors)
bool wgrad_uniform_tap(const ConvP& p) {
  // (byte offsets into x and dzdy stay below the "outside" offset of the buffer loads)
  return p.FC % 32 == 0 && (long long)p.H * p.W * p.C * p.N < (1ll << 29) &&
         (long long)p.outH * p.outW * p.K * p.N < (1ll << 29) && !tunable("conv_no_uniform_tap", 0);
}

// filter-volume rows per workgroup of the filter-gradient kernel: 128; 64 when the whole volume fits in 64 rows (a
// 1x1 layer with 64 input channels) and the filter tile leaves room for that shape; 192 when a volume of 129...192
// rows meets a 64-filter tile (the 7x7x3 = 147-row stem of ResNet-50: one tile instead of two, dzdy read once:
// 201 -> 150 us at 32 images)
int pick_rows_tile(const ConvP& p) {
  const int FV = p.FH * p.FW * p.FC, BA = pick_channels_tile(p.K);
  if (FV <= 64 && BA >= 64) return 64;
  if (FV > 128 && FV <= 192 && BA == 64 && !tunable("conv_wgrad_no_wide_rows", 0)) return 192;
  // a volume that 192-row tiles cover exactly and 128-row tiles do not (3x3x64 = 576 rows: three tiles instead of
  // four and a half, and 48 instead of 32 MFMAs per wavefront between two barriers)
  if (FV % 192 == 0 && FV % 128 != 0 && BA == 64) return 192;
  return 128;
}

int wgrad_splits(const ConvP& p, int* tilesOut) {
  const int BA = pick_channels_tile(p.K), BB = pick_rows_tile(p);
  const int tiles = ((p.K + BA - 1) / BA) * ((p.FH * p.FW * p.FC + BB - 1) / BB);
  // two workgroups per CU; one when a workgroup's share of a 1x1 layer would be under ~10 MFLOP with several tiles
  // to write (the partial banks then cost more than the idle half: 14x14 and 7x7 1x1 layers of ResNet-50 at 32
  // images 46.6 -> 44.8 us, 54.6 -> 50.0 us), or when the whole bank is one tile
  const double flops = 2.0 * p.outH * p.outW * p.N * (double)p.FH * p.FW * p.FC * p.K;
  const bool small1x1 = p.FH * p.FW == 1 && flops < 5e9 && (tiles >= 4 || tiles == 1);
  const int target = small1x1 ? 256 : 512;
  const long long chunks = ((long long)p.outH * p.outW * p.N + 31) / 32;
  long long s = std::max<long long>(1, target / tiles);
  s = std::min<long long>(s, std::max<long long>(1, chunks / 4));  // at least 4 reduction steps per split
  if (tilesOut) *tilesOut = tiles;
  return (int)s;
}

template <int WA, int WB, int NWA, int NWB>
void launch_pix(hipStream_t s, float* out, const float* in, const float* wt, const float* bias, const PixP& p, bool ut) {
  constexpr int BA = WA * 32 * NWA, BB = WB * 32 * NWB;
  const long long mTiles = ((long long)p.M + BB - 1) / BB;
  const int tilesA = (p.Cout + BA - 1) / BA;
  const dim3 grid((unsigned)(mTiles * tilesA * p.rSplits));
  KernelTimer timer("conv_pix_mfma", s);
  if constexpr (BA >= 64 && BB >= 64) {
    if (ut && p.inBytes != 0 && p.wtBytes != 0) {
      hipLaunchKernelGGL((conv_pix_mfma<WA, WB, NWA, NWB, true, true>), grid, dim3(256), 3 * 16 * (BA + BB) * sizeof(float) + kMaxTaps * sizeof(int2), s, out,
                         in, wt, bias, p);
      return;
    }
  }
  if (ut) hipLaunchKernelGGL((conv_pix_mfma<WA, WB, NWA, NWB, true>), grid, dim3(256), 0, s, out, in, wt, bias, p);
  else hipLaunchKernelGGL((conv_pix_mfma<WA, WB, NWA, NWB, false>), grid, dim3(256), 0, s, out, in, wt, bias, p);
}

// `shape` as in PixPlan; the tunable forces one for experiments (it must fit the channel tile)
void launch_shape(hipStream_t s, int shape, float* out, const float* in, const float* wt, const float* bias, const PixP& p,
                  bool ut) {
  const int BA = pick_channels_tile(p.Cout);
  if ((shape == 1 || shape == 5 || shape == 7) && BA != 128) shape = BA == 64 ? 2 : 3;
  if ((shape == 2 || shape == 4 || shape == 6) && BA != 64) shape = BA == 128 ? 1 : 3;
  if (shape == 3 && BA != 32) shape = BA == 128 ? 1 : 2;
  switch (shape) {
    case 1: launch_pix<2, 2, 2, 2>(s, out, in, wt, bias, p, ut); break;  // 128 x 128
    case 2: launch_pix<2, 2, 1, 4>(s, out, in, wt, bias, p, ut); break;  //  64 x 256
    case 3: launch_pix<1, 2, 1, 4>(s, out, in, wt, bias, p, ut); break;  //  32 x 256
    case 4: launch_pix<1, 2, 2, 2>(s, out, in, wt, bias, p, ut); break;  //  64 x 128
    case 5: launch_pix<2, 1, 2, 2>(s, out, in, wt, bias, p, ut); break;  // 128 x  64
    case 7: launch_pix<1, 1, 4, 1>(s, out, in, wt, bias, p, ut); break;  // 128 x  32
    default: launch_pix<1, 1, 2, 2>(s, out, in, wt, bias, p, ut); break; //  64 x  64
  }
}

template <int WA, int WB, int NWA, int NWB, bool UT, bool DIRECT = false, bool DEEP = false>
int launch_wgrad(hipStream_t s, dim3 grid, float* out, const float* x, const float* dy, const WgP& p) {
  constexpr int BA = WA * 32 * NWA, BB = WB * 32 * NWB, LD = 33;
  constexpr size_t lds = (size_t)wgrad_buffers(BA, BB, DIRECT, DEEP) * (BA + BB) * LD * sizeof(float) + BB * sizeof(int2);
  static std::atomic<bool> raisedOn[kMaxDevices];  // opt-in to more than 64 KB of LDS per workgroup, once per device
  const int dev = current_device();
  const bool raised = dev >= 0 && dev < kMaxDevices && raisedOn[dev].load(std::memory_order_acquire);
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)conv_wgrad_mfma<WA, WB, NWA, NWB, UT, DIRECT, DEEP>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return fail(MCN_DEVICE_ERROR, "mcn_conv_backward_filter: cannot reserve %zu bytes of LDS", lds);
    }
    if (dev >= 0 && dev < kMaxDevices) raisedOn[dev].store(true, std::memory_order_release);
  }
  // On a stream marked as running beside another one the launch asks for more local memory than it uses, so that a CU
  // holds one of its workgroups at a time and the other stream's kernels keep the rest of the CU.
  size_t ldsAsk = lds;
  if (stream_beside(s)) {
    ldsAsk = std::max(lds, (size_t)84 * 1024);
    static std::atomic<bool> widened[kMaxDevices];
    if (ldsAsk > 64 * 1024 && ldsAsk > lds && dev >= 0 && dev < kMaxDevices && !widened[dev].load(std::memory_order_acquire)) {
      if (hipFuncSetAttribute((const void*)conv_wgrad_mfma<WA, WB, NWA, NWB, UT, DIRECT, DEEP>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              128 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        ldsAsk = lds;  // (the launch goes ahead with what it needs)
      } else {
        widened[dev].store(true, std::memory_order_release);
      }
    }
  }
  KernelTimer timer("conv_wgrad_mfma", s);
  hipLaunchKernelGGL((conv_wgrad_mfma<WA, WB, NWA, NWB, UT, DIRECT, DEEP>), grid, dim3(256), ldsAsk, s, out, x, dy, p);
  return MCN_SUCCESS;
}

// Tile shape of the tiled kernel (channels x pixels per workgroup) and how many ways the reduction is split.
struct PixPlan {
  int shape;   // 1: 128x128  2: 64x256  3: 32x256  4: 64x128  5: 128x64  6: 64x64  7: 128x32
  int splits;
};

PixPlan plan_pix(int Cout, long long M, int R) {
  PixPlan plan;
  const int BA = pick_channels_tile(Cout);
  const long long tilesA = (Cout + BA - 1) / BA;
  auto blocks = [&](int px) { return ((M + px - 1) / px) * tilesA; };
  // the widest pixel tile that still yields >= 2048 workgroups (8 per CU), because short reduction loops hide
  // their load latency only through occupancy
  int px;
  if (BA == 128) { plan.shape = M <= 32 ? 7 : (blocks(128) >= 2048 ? 1 : 5); px = plan.shape == 7 ? 32 : (plan.shape == 1 ? 128 : 64); }
  else if (BA == 64) { plan.shape = blocks(256) >= 2048 ? 2 : (blocks(128) >= 2048 ? 4 : 6); px = plan.shape == 2 ? 256 : (plan.shape == 4 ? 128 : 64); }
  else { plan.shape = 3; px = 256; }
  // fewer than two workgroups per CU with a long reduction each: split it, down to 12 steps of 16 rows per
  // workgroup.  How many ways: the count with the least modelled time -- the busiest CU's workgroups (dealt evenly)
  // times their steps at the rate that many resident workgroups reach, plus the partial results written and read
  // back once per split.  What
  // matters at these sizes is how the workgroups divide among the CUs (196 tiles on 256 CUs: 5 splits leave at most 4
  // workgroups of 29 steps on a CU, 6 splits 5 of 24; 3x3x256x256 on 14x14x256x32 82 -> 76 us, 3x3x512x512 on
  // 7x7x512x32 95 -> 84 us).
  plan.splits = 1;
  const long long nb = blocks(px);
  const int nSteps = (R + 15) / 16;
  const int maxBlocks = 512, minSteps = 12;
  if (nb <= maxBlocks && nSteps >= 4 * minSteps && !tunable("conv_no_split", 0)) {
    const int cus = std::max(1, device_compute_units());
    const double stepUs = 32.0 * BA * px / (157.3e6 / 256.0);           // one step of one tile on one CU
    const double partUs = 2.0 * (double)M * Cout * sizeof(float) / 5e6;  // one split's partial results, out and back
    double best = 0;
    for (int s = 1; s <= std::min(nSteps / minSteps, 16); ++s) {
      // (a CU's workgroups share its matrix pipes; with few of them the pipes wait for loads and barriers: rates measured
      // on 3x3x256x256 over 14x14x256x32 with 1, 2, 3 and 4 workgroups to a CU)
      static const double rate[5] = {0, 0.63, 0.80, 0.85, 0.88};
      const long long perCu = (nb * s + cus - 1) / cus;
      const double cost = (double)perCu * ((nSteps + s - 1) / s) * stepUs / rate[std::min<long long>(perCu, 4)] + (s > 1 ? s * partUs + 6.0 : 0.0);
      if (s == 1 || cost < best) { best = cost; plan.splits = s; }
    }
  }
  return plan;
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

// (run_pix with a PixCollect: the product is not launched but appended to a launch of several; wsUsed reports what its
// bank, packed on the fly, takes of the workspace)
struct PixCollect {
  PixMulti m;
  size_t wsUsed;
};

int run_pix(hipStream_t s, const char* who, float* out, const float* in, const float* f, const float* bias, PixP p,
            const TapSet& taps, int backward, void* ws, size_t wsBytes, PackCtx* pk, PixCollect* collect = nullptr) {
  const int BA = pick_channels_tile(p.Cout);
  const int rPad = (p.R + 15) / 16 * 16;
  p.coutPad = (p.Cout + BA - 1) / BA * BA;
  const PixPlan plan = plan_pix(p.Cout, p.M, p.R);
  const size_t nOut = (size_t)p.N * p.Cout * p.OH * p.OW;
  const size_t needW = (size_t)rPad * p.coutPad * sizeof(float);
  // uniform-tap variant: whole 16-row steps inside one tap, and 32-bit element offsets into the gathered tensor
  const long long inSpan = (long long)(p.N - 1) * p.inImg + (long long)p.Cin * p.IH * p.IW;  // elements from `in` to the end
  const bool ut = p.Cin % 16 == 0 && inSpan < (1ll << 31) && !tunable("conv_no_uniform_tap", 0);
  {
    const long long ob = ((long long)(p.N - 1) * p.outImg + (long long)p.Cout * p.outPlane) * 4;
    p.outBytes = ob < (1ll << 31) ? (unsigned)ob : 0u;
  }
  if (p.statQuery) {  // (plan only: would this product also sum its output per channel, and into how many partials?)
    *p.statQuery = ut && p.Cout > 4 && !bias && p.beta == 0.f ? conv_ws_stat_groups(p) : 0;
    return MCN_SUCCESS;
  }
  if (p.stats && !(ut && p.Cout > 4)) return fail(MCN_UNSUPPORTED, "%s: this product cannot sum its output per channel", who);
  if (p.addQuery) {  // (plan only: can this product add a masked second term in its epilogue?)
    *p.addQuery = 0;
    if (ut && p.Cout > 4) {
      int handled = 0;
      return conv_ws_launch(s, who, out, in, nullptr, bias, p, &handled);
    }
    return MCN_SUCCESS;
  }
  if (p.addend && !(ut && p.Cout > 4)) return fail(MCN_UNSUPPORTED, "%s: this product cannot add a masked second term in its epilogue", who);
  // The backward-data product of a 1x1 bank whose extents need no padding reads it as it is stored: rows = filters,
  // columns = the filters' channels, which is the packed order.
  const bool asStored = backward && taps.FH * taps.FW == 1 && rPad == p.R && p.coutPad == p.Cout && aligned16(f);
  float* slot = nullptr;  // this bank's place in a buffer packed ahead
  if (pk && !asStored) {
    slot = pk->base ? (float*)(pk->base + pk->offset) : nullptr;
    pk->offset += align256(needW);
    if (pk->mode != PackCtx::kPlan && pk->offset > pk->capacity)
      return fail(MCN_ILLEGAL_ARGUMENT, "%s: packed filter buffer too small (%zu < %zu bytes)", who, pk->capacity, pk->offset);
  }
  if (pk && pk->mode != PackCtx::kUse) {
    if (asStored) return MCN_SUCCESS;
    if (pk->mode == PackCtx::kPlan) {
      if (pk->jobs) {
        PackJob j;
        j.wt = slot; j.f = f; j.taps = taps;
        j.Cin = p.Cin; j.Cout = p.Cout; j.rPad = rPad; j.coutPad = p.coutPad; j.backward = backward; j.tapMajor = pack_flags(taps, backward, ut, rPad, p.coutPad, true);
        j.firstBlock = 0; j.blocks = pack_blocks(j.tapMajor, rPad, p.coutPad);
        pk->jobs->push_back(j);
      }
      return MCN_SUCCESS;
    }
    KernelTimer timer("conv_pack_weights", s);
    const int flags = pack_flags(taps, backward, ut, rPad, p.coutPad, false);
    hipLaunchKernelGGL(conv_pack_weights, dim3(pack_blocks(flags, rPad, p.coutPad)), dim3(256), 0, s, slot, f, taps, p.Cin, p.Cout,
                       rPad, p.coutPad, backward, flags);
    return check_launch(who);
  }
  int sbSplits = 1;
  const bool sb = ut && p.Cout > 4 && !p.stats && conv_sb_plan(p, &sbSplits);
  const int needSplits = std::max(plan.splits, sb ? sbSplits : 1);
  const size_t tailBytes = sb && sbSplits == 1 ? conv_sb_tail_bytes(p.Cout, p.M, p.R) : 0;
  // The partial tensors of a split reduction must fit; the scratch for the left-over tiles of the streamed-bank kernel is
  // taken when the workspace has room for it and done without otherwise (every tile by one workgroup): a workspace
  // sized before a tunable changed, or fixed for a captured graph, stays valid.
  const size_t needParts = needSplits > 1 ? (size_t)needSplits * nOut * sizeof(float) : (size_t)0;
  const size_t need = needParts && !collect ? align256(needW) + needParts : (slot || asStored ? 0 : needW);
  if (collect) collect->wsUsed = slot || asStored ? 0 : align256(needW);
  if (need && (!ws || wsBytes < need)) return fail(MCN_ILLEGAL_ARGUMENT, "%s: workspace too small (%zu < %zu bytes)", who, wsBytes, need);
  if (need && !aligned16(ws)) return fail(MCN_ILLEGAL_ARGUMENT, "%s: workspace must be 16-byte aligned", who);
  const bool haveTail = tailBytes && ws && aligned16(ws) && wsBytes >= align256(needW) + tailBytes;
  float* wt = (float*)ws;
  int rc = MCN_SUCCESS;
  if (asStored) {
    wt = const_cast<float*>(f);
  } else if (slot) {
    wt = slot;
  } else {
    KernelTimer timer("conv_pack_weights", s);
    const int flags = pack_flags(taps, backward, ut, rPad, p.coutPad, false);
    hipLaunchKernelGGL(conv_pack_weights, dim3(pack_blocks(flags, rPad, p.coutPad)), dim3(256), 0, s, wt, f, taps, p.Cin, p.Cout,
                       rPad, p.coutPad, backward, flags);
    rc = check_launch(who);
  }
  if (rc) return rc;
  if (((long long)p.M / 64 + 1) * (p.coutPad / 32) >= (1ll << 31)) return fail(MCN_UNSUPPORTED, "%s: tensor too large", who);
  {
    const long long ob = ((long long)(p.N - 1) * p.outImg + (long long)p.Cout * p.outPlane) * 4;
    p.outBytes = ob < (1ll << 31) ? (unsigned)ob : 0u;
  }
  {
    // (loads straight into LDS in the tiled kernel: both operands behind buffer descriptors of less than 2 GiB)
    const long long ib = inSpan * 4, wb = (long long)rPad * p.coutPad * 4;
    const bool direct = ut && ib < (1ll << 31) && wb < (1ll << 31);
    p.inBytes = direct ? (unsigned)ib : 0u;
    p.wtBytes = direct ? (unsigned)wb : 0u;
  }
  p.byQ = FastDiv(p.OH * p.OW);
  p.byOH = FastDiv(p.OH);
  p.byT = FastDiv(p.T);
  p.advC = 16 / p.T;
  p.advT = 16 % p.T;
  p.rSplits = 1;
  p.stepsPerSplit = 0;
  p.partStride = 0;
  if (collect) {
    if (!p.inBytes || !p.wtBytes || collect->m.n >= kMaxMulti) return fail(MCN_UNSUPPORTED, "%s: product cannot join a launch of several", who);
    collect->m.p[collect->m.n] = p;
    collect->m.wt[collect->m.n] = wt;
    ++collect->m.n;
    return MCN_SUCCESS;
  }
  // one to four output channels (the input gradient of a first layer): conv_few.hip
  if (p.Cout <= 4) {
    int handled = 0;
    rc = conv_few_launch(s, who, out, in, wt, bias, p, ut, &handled);
    if (rc || handled) return rc;
  }
  // small filter banks: keep all the weights in LDS and stream the pixels past them (conv_ws.hip)
  if (ut) {
    int handled = 0;
    rc = conv_ws_launch(s, who, out, in, wt, bias, p, &handled);
    if (rc || handled) return rc;
  }
  if (p.stats) return fail(MCN_UNSUPPORTED, "%s: this product cannot sum its output per channel", who);
  if (p.addend) return fail(MCN_UNSUPPORTED, "%s: this product cannot add a masked second term in its epilogue", who);
  // banks too large for LDS: stream them past pixels held in registers (conv_sb.hip)
  if (sb && sbSplits == 1) {
    rc = conv_sb_launch(s, out, in, wt, bias, p, 1, haveTail ? (float*)((char*)ws + align256(needW)) : nullptr);
    return rc ? rc : check_launch(who);
  }
  if (sb || plan.splits > 1) {
    // every workgroup a slice of the reduction into its own partial tensor, then one pass to add them up
    float* partials = (float*)((char*)ws + align256(needW));
    PixP q = p;
    const int nSteps = rPad / 16;
    q.stepsPerSplit = (nSteps + plan.splits - 1) / plan.splits;
    q.rSplits = sb ? sbSplits : (nSteps + q.stepsPerSplit - 1) / q.stepsPerSplit;
    q.partStride = (long long)nOut;
    q.alpha = 1.f;
    q.beta = 0.f;
    // the partial tensors are dense whatever the destination's layout is
    q.outPlane = q.OH * q.OW;
    q.outImg = q.Cout * q.outPlane;
    q.outOff = 0; q.outSH = 1; q.outSW = q.OH; q.dense = 1;
    {
      const long long ob = (long long)nOut * 4;
      q.outBytes = ob < (1ll << 31) ? (unsigned)ob : 0u;
    }
    if (sb) rc = conv_sb_launch(s, partials, in, wt, nullptr, q, sbSplits, nullptr);
    else launch_shape(s, plan.shape, partials, in, wt, nullptr, q, ut);
    if (rc || (rc = check_launch(who))) return rc;
    p.rSplits = q.rSplits;
    p.partStride = q.partStride;
    KernelTimer timer("conv_pix_reduce", s);
    const FastDiv byCout(p.Cout);
    const bool flat = p.dense != 0 && p.outImg == p.Cout * p.outPlane && nOut % 4 == 0 && nOut < (1ull << 31) &&
                      aligned16(out) && aligned16(partials);
    if (flat)
      hipLaunchKernelGGL((conv_pix_reduce<true, false>), dim3((unsigned)((nOut / 4 + 255) / 256)), dim3(256), 0, s, out,
                         partials, bias, nOut, p, byCout);
    else if (nOut < (1ull << 31))
      hipLaunchKernelGGL((conv_pix_reduce<false, false>), dim3((unsigned)((nOut + 255) / 256)), dim3(256), 0, s, out,
                         partials, bias, nOut, p, byCout);
    else
      hipLaunchKernelGGL((conv_pix_reduce<false, true>), dim3((unsigned)((nOut + 255) / 256)), dim3(256), 0, s, out,
                         partials, bias, nOut, p, byCout);
    return check_launch(who);
  }
  launch_shape(s, plan.shape, out, in, wt, bias, p, ut);
  return check_launch(who);
}

int gcd_int(int a, int b) { return b == 0 ? a : gcd_int(b, a % b); }

// One axis of a stride class of the backward-data product (see backward_data_group): the taps that take part are
// first, first + step, ... (count of them); the gathered position starts at dBase and moves by dStep per tap.
struct Axis { int first, step, count, dBase, dStep; };
Axis stride_axis(int phase, int pad, int dil, int stride, int taps) {
  Axis a;
  a.step = stride / gcd_int(dil, stride);
  a.first = -1;
  for (int i = 0; i < taps && i < a.step; ++i)
    if ((phase + pad - i * dil) % stride == 0) { a.first = i; break; }
  a.count = a.first < 0 ? 0 : (taps - a.first + a.step - 1) / a.step;
  a.dBase = a.first < 0 ? 0 : (phase + pad - a.first * dil) / stride;  // exact: the numerator is a multiple of stride
  a.dStep = -(a.step * dil) / stride;                                   // exact likewise
  return a;
}

// The stride classes of a strided layer's backward-data product in ONE launch of the tiled kernel (conv_pix_multi) instead
// of one launch each: every class is a quarter of the work with a launch's fixed costs to itself, and at network sizes
// those costs are most of it (3x3 /2, 256 -> 256 onto 28x28x256x32: four launches and a fill, 121 us; one launch ...).
// Whether a layer (one filter group of it) takes this path depends on its geometry only: 2...4 classes with taps,
// channels in whole steps of 16, tiles of at least 64 channels, tensors within 32-bit byte offsets, not more tiles than
// leave a launch per class short.  Returns the number of classes, 0 = one launch per class.
int multi_classes(const ConvP& p, Wide wd, size_t* bankBytes) {
  if (bankBytes) *bankBytes = 0;
  if ((p.sy == 1 && p.sx == 1) || !tunable("conv_pix_multi", 1)) return 0;
  if (p.K % 16 != 0 || tunable("conv_no_uniform_tap", 0)) return 0;
  const long long inSpan = (long long)(p.N - 1) * wd.yImg + (long long)p.K * p.outH * p.outW;
  if (inSpan * 4 >= (1ll << 31)) return 0;
  const int BA = pick_channels_tile(p.C);
  if (BA < 64) return 0;
  const long long tilesA = (p.C + BA - 1) / BA, coutPad = tilesA * BA;
  int n = 0;
  long long tiles = 0;
  size_t banks = 0;
  for (int pw = 0; pw < p.sx && pw < p.W; ++pw)
    for (int ph = 0; ph < p.sy && ph < p.H; ++ph) {
      const Axis ai = stride_axis(ph, p.pt, p.dy, p.sy, p.FH), aj = stride_axis(pw, p.pl, p.dx, p.sx, p.FW);
      if (ai.count == 0 || aj.count == 0) continue;
      ++n;
      const long long M = (long long)((p.H - ph + p.sy - 1) / p.sy) * ((p.W - pw + p.sx - 1) / p.sx) * p.N;
      const long long bank = (long long)ai.count * aj.count * p.K * coutPad * 4;  // (K a multiple of 16: no padded rows)
      if (bank >= (1ll << 31)) return 0;
      banks += align256((size_t)bank);
      tiles += (M + 63) / 64 * tilesA;
    }
  if (n < 2 || n > kMaxMulti || tiles > 4096) return 0;
  if (bankBytes) *bankBytes = banks;
  return n;
}

template <int WA, int WB, int NWA, int NWB>
void launch_multi(hipStream_t s, float* out, const float* in, PixMulti& m) {
  constexpr int BA = WA * 32 * NWA, BB = WB * 32 * NWB;
  unsigned at = 0;
  for (int i = 0; i < m.n; ++i) {
    m.first[i] = at;
    at += (unsigned)((((long long)m.p[i].M + BB - 1) / BB) * ((m.p[i].Cout + BA - 1) / BA));
  }
  for (int i = m.n; i <= kMaxMulti; ++i) m.first[i] = at;
  KernelTimer timer("conv_pix_multi", s);
  hipLaunchKernelGGL((conv_pix_multi<WA, WB, NWA, NWB>), dim3(at), dim3(256), 3 * 16 * (BA + BB) * sizeof(float) + kMaxTaps * sizeof(int2), s,
                     out, in, m);
}

}  // namespace

bool conv_mfma_forward_supported(const ConvP& p) { return common_ok(fc_view(p)); }
bool conv_mfma_backward_data_supported(const ConvP& p) { return common_ok(fc_view(p)); }
bool conv_mfma_backward_filter_supported(const ConvP& p) { return common_ok(fc_view(p)); }

size_t conv_mfma_workspace_bytes(const ConvP& original, int product) {
  const ConvP layer = fc_view(original);
  const ConvP p = group_view(layer);  // the groups run one after the other through the same workspace
  const size_t FV = (size_t)p.FH * p.FW * p.FC;
  // packed bank, plus the partial results when the tiled kernel splits the reduction (plan_pix)
  auto pix_need = [&](int Cout, long long M, int R) {
    const int BA = pick_channels_tile(Cout);
    const size_t needW = ((size_t)(R + 15) / 16 * 16) * (size_t)((Cout + BA - 1) / BA * BA) * sizeof(float);
    const PixPlan plan = plan_pix(Cout, M, R);
    const int splits = std::max(plan.splits, conv_sb_splits(Cout, M, R));  // (whichever kernel takes the product)
    const size_t parts = std::max(splits > 1 ? (size_t)splits * (size_t)M * Cout * sizeof(float) : (size_t)0,
                                  conv_sb_tail_bytes(Cout, M, R));
    return parts ? align256(needW) + parts : needW;
  };
  switch (product) {
    case MCN_CONV_FORWARD: {
      if (!conv_mfma_forward_supported(layer)) return 0;
      return pix_need(p.K, (long long)p.outH * p.outW * p.N, (int)FV);
    }
    case MCN_CONV_BACKWARD_DATA: {
      if (!conv_mfma_backward_data_supported(layer)) return 0;
      // all classes in one launch: their banks side by side
      size_t banks = 0;
      if (multi_classes(p, wide_of(layer), &banks)) return banks;
      // the largest need of any stride class (one class, all taps, when the strides are 1)
      size_t need = 0;
      for (int pw = 0; pw < p.sx && pw < p.W; ++pw)
        for (int ph = 0; ph < p.sy && ph < p.H; ++ph) {
          const Axis ai = stride_axis(ph, p.pt, p.dy, p.sy, p.FH), aj = stride_axis(pw, p.pl, p.dx, p.sx, p.FW);
          if (ai.count == 0 || aj.count == 0) continue;
          const long long M = (long long)((p.H - ph + p.sy - 1) / p.sy) * ((p.W - pw + p.sx - 1) / p.sx) * p.N;
          need = std::max(need, pix_need(p.C, M, ai.count * aj.count * p.K));
        }
      return need;
    }
    case MCN_CONV_BACKWARD_FILTER: {
      if (!conv_mfma_backward_filter_supported(layer)) return 0;
      const int s = wgrad_splits(p, nullptr);
      return (s > 1 || wgrad_uniform_tap(layer)) ? (size_t)s * FV * p.K * sizeof(float) : 0;
    }
    default: return 0;
  }
}

namespace {

TapSet all_taps(const ConvP& p) {
  TapSet t;
  t.FH = p.FH; t.FW = p.FW;
  t.i0 = 0; t.iStep = 1; t.nI = p.FH;
  t.j0 = 0; t.jStep = 1; t.nJ = p.FW;
  return t;
}

void dense_layout(PixP* q) {
  q->inImg = q->Cin * q->IH * q->IW;
  q->outPlane = q->OH * q->OW;
  q->outImg = q->Cout * q->outPlane;
  q->outOff = 0; q->outSH = 1; q->outSW = q->OH; q->dense = 1;
}


}  // namespace

namespace {
int forward_group(hipStream_t s, const ConvP& p, Wide wd, float* y, float outMult, const float* x, float inMult,
                  const float* f, const float* b, void* ws, size_t wsBytes, PackCtx* pk, double* stats, int statGroups,
                  int* statQuery) {
  PixP q;
  q.stats = stats;
  q.statGroups = statGroups;
  q.statQuery = statQuery;
  q.IH = p.H; q.IW = p.W; q.Cin = p.C;
  q.OH = p.outH; q.OW = p.outW; q.Cout = p.K;
  q.N = p.N;
  q.FH = p.FH; q.T = p.FH * p.FW;
  q.sy = p.sy; q.sx = p.sx;
  q.dhBase = -p.pt; q.dhStep = p.dy; q.dwBase = -p.pl; q.dwStep = p.dx;
  q.R = q.T * q.Cin;
  q.coutPad = 0;
  q.M = p.outH * p.outW * p.N;
  q.alpha = inMult; q.beta = outMult;
  dense_layout(&q);
  q.inImg = wd.xImg;
  q.outImg = wd.yImg;
  return run_pix(s, "mcn_conv_forward", y, x, f, b, q, all_taps(p), 0, ws, wsBytes, pk);
}
}  // namespace

int conv_pack_batch(hipStream_t s, const PackJob* deviceJobs, int nJobs, unsigned totalBlocks) {
  if (nJobs <= 0 || totalBlocks == 0) return MCN_SUCCESS;
  KernelTimer timer("conv_pack_many", s);
  hipLaunchKernelGGL(conv_pack_many, dim3(totalBlocks), dim3(256), 0, s, deviceJobs, nJobs);
  return check_launch("mcn_conv_pack_batch");
}

int conv_forward_mfma(hipStream_t s, const ConvP& original, float* y, float outMult, const float* x, float inMult,
                      const float* f, const float* b, void* ws, size_t wsBytes, PackCtx* pk, double* stats, int statGroups,
                      int* statQuery) {
  const ConvP p = fc_view(original);
  const ConvP g = group_view(p);
  const Wide wd = wide_of(p);
  if ((stats || statQuery) && p.groups != 1) {
    if (statQuery) {
      *statQuery = 0;
      return MCN_SUCCESS;
    }
    return fail(MCN_UNSUPPORTED, "mcn_conv_forward_sums: filter groups are not supported");
  }
  const size_t FV = (size_t)p.FH * p.FW * p.FC, Q = (size_t)p.outH * p.outW, HW = (size_t)p.H * p.W;
  for (int i = 0; i < p.groups; ++i) {
    int rc = forward_group(s, g, wd, y + i * p.Kg * Q, outMult, x + i * p.FC * HW, inMult, f + i * p.Kg * FV,
                           b ? b + i * p.Kg : nullptr, ws, wsBytes, pk, stats, statGroups, statQuery);
    if (rc) return rc;
  }
  return MCN_SUCCESS;
}

// dzdx[h, w] = sum over taps (i, j) with (h + pt - i*dy) and (w + pl - j*dx) divisible by the strides of
//   dzdy[(h + pt - i*dy)/sy, (w + pl - j*dx)/sx] * f[i, j]
// With unit stride that is one gather product over all taps.  With a stride the pixels split into sy*sx classes
// (h mod sy, w mod sx); inside a class the taps that take part form an arithmetic progression and the gathered
// position moves by one per pixel of the class, so each class is the same gather product over a sub-grid of dzdx
// with a subset of the taps.  Classes no tap reaches (1x1 filters with stride 2: three of four) are zeros.
namespace {
int backward_data_group(hipStream_t s, const ConvP& p, Wide wd, float* dx, float dxMult, const float* f, const float* dy,
                        void* ws, size_t wsBytes, PackCtx* pk, const float* addend, const unsigned* addBits, int* addQuery) {
  PixP q;
  q.addend = addend;
  q.addBits = addBits;
  q.addQuery = addQuery;
  q.IH = p.outH; q.IW = p.outW; q.Cin = p.K;
  q.N = p.N;
  q.Cout = p.C;
  q.sy = 1; q.sx = 1;
  q.coutPad = 0;
  q.alpha = 1.f; q.beta = dxMult;
  if (p.sy == 1 && p.sx == 1) {
    q.OH = p.H; q.OW = p.W;
    q.FH = p.FH; q.T = p.FH * p.FW;
    q.dhBase = p.pt; q.dhStep = -p.dy; q.dwBase = p.pl; q.dwStep = -p.dx;
    q.R = q.T * q.Cin;
    q.M = p.H * p.W * p.N;
    dense_layout(&q);
    q.inImg = wd.yImg;
    q.outImg = wd.xImg;
    return run_pix(s, "mcn_conv_backward_data", dx, dy, f, nullptr, q, all_taps(p), 1, ws, wsBytes, pk);
  }
  // one class at a time (the caller has dealt with the classes no tap reaches), or all of them in one launch.  Either way
  // the classes with the most taps go first: in a shared launch the longest workgroups should start first, and planning,
  // packing and using the banks must walk the classes in one order whichever way the launches go.
  const int together = multi_classes(p, wd, nullptr);
  PixCollect batch;
  batch.m.n = 0;
  size_t wsAt = 0;
  for (int most = p.FH * p.FW; most >= 1; --most)
  for (int pw = 0; pw < p.sx && pw < p.W; ++pw)
    for (int ph = 0; ph < p.sy && ph < p.H; ++ph) {
      const Axis ai = stride_axis(ph, p.pt, p.dy, p.sy, p.FH), aj = stride_axis(pw, p.pl, p.dx, p.sx, p.FW);
      if (ai.count * aj.count != most) continue;
      PixP c = q;
      c.OH = (p.H - ph + p.sy - 1) / p.sy;
      c.OW = (p.W - pw + p.sx - 1) / p.sx;
      c.FH = ai.count; c.T = ai.count * aj.count;
      c.dhBase = ai.dBase; c.dhStep = ai.dStep; c.dwBase = aj.dBase; c.dwStep = aj.dStep;
      c.R = c.T * c.Cin;
      c.M = c.OH * c.OW * p.N;
      c.inImg = wd.yImg;
      c.outPlane = p.H * p.W;
      c.outImg = wd.xImg;
      c.outOff = ph + p.H * pw; c.outSH = p.sy; c.outSW = p.H * p.sx; c.dense = 0;
      TapSet t;
      t.FH = p.FH; t.FW = p.FW;
      t.i0 = ai.first; t.iStep = ai.step; t.nI = ai.count;
      t.j0 = aj.first; t.jStep = aj.step; t.nJ = aj.count;
      int rc;
      if (together) {
        batch.wsUsed = 0;
        rc = run_pix(s, "mcn_conv_backward_data", dx, dy, f, nullptr, c, t, 1, ws ? (char*)ws + wsAt : nullptr,
                     wsBytes > wsAt ? wsBytes - wsAt : 0, pk, &batch);
        wsAt += batch.wsUsed;
      } else {
        rc = run_pix(s, "mcn_conv_backward_data", dx, dy, f, nullptr, c, t, 1, ws, wsBytes, pk);
      }
      if (rc) return rc;
    }
  if (together && batch.m.n > 0) {
    // 128 x 64 tiles, or 64 channels x 128 or 64 pixels: the smaller ones while the larger would leave fewer than two
    // tiles to a CU (the classes' reductions differ four to one in length: with few tiles the longest sets the time)
    long long tiles128 = 0, tilesWide = 0;
    for (int i = 0; i < batch.m.n; ++i) {
      tiles128 += ((long long)batch.m.p[i].M + 127) / 128;
      tilesWide += (((long long)batch.m.p[i].M + 63) / 64) * ((p.C + 127) / 128);
    }
    const int few = 2 * std::max(1, device_compute_units());
    if (pick_channels_tile(p.C) == 128 && tilesWide >= few) launch_multi<2, 1, 2, 2>(s, dx, dy, batch.m);
    else if (tiles128 >= 512) launch_multi<1, 2, 2, 2>(s, dx, dy, batch.m);
    else launch_multi<1, 1, 2, 2>(s, dx, dy, batch.m);
    return check_launch("mcn_conv_backward_data");
  }
  return MCN_SUCCESS;
}
}  // namespace

int conv_backward_data_mfma(hipStream_t s, const ConvP& original, float* dx, float dxMult, const float* f, const float* dy,
                            void* ws, size_t wsBytes, PackCtx* pk, const float* addend, const unsigned* addBits, int* addQuery) {
  const ConvP p = fc_view(original);
  if (addend || addQuery) {
    // the masked second term: one product over the whole tensor (no filter groups, no stride classes)
    if (p.groups != 1 || p.sy != 1 || p.sx != 1 || dxMult != 0.f) {
      if (addQuery) {
        *addQuery = 0;
        return MCN_SUCCESS;
      }
      return fail(MCN_UNSUPPORTED, "mcn_conv_backward_data_masked_add: not available for this geometry");
    }
    return backward_data_group(s, group_view(p), wide_of(p), dx, 0.f, f, dy, ws, wsBytes, pk, addend, addBits, addQuery);
  }
  const bool compute = !pk || pk->mode == PackCtx::kUse;
  // stride classes no tap reaches get no launch: they are zeros (or keep what is there, when accumulating)
  bool anyEmpty = false;
  for (int pw = 0; pw < p.sx && pw < p.W; ++pw)
    for (int ph = 0; ph < p.sy && ph < p.H; ++ph)
      if (stride_axis(ph, p.pt, p.dy, p.sy, p.FH).count == 0 || stride_axis(pw, p.pl, p.dx, p.sx, p.FW).count == 0) anyEmpty = true;
  if (!compute) {
  } else if (anyEmpty && dxMult == 0.f) {
    int rc = mcn_fill((mcn_stream_t)s, dx, 0.f, (size_t)p.H * p.W * p.C * p.N);
    if (rc) return rc;
  } else if (anyEmpty && dxMult != 1.f) {
    return fail(MCN_UNSUPPORTED, "mcn_conv_backward_data: accumulation with a multiplier other than 1 is not available for this stride");
  }
  const ConvP g = group_view(p);
  const Wide wd = wide_of(p);
  const size_t FV = (size_t)p.FH * p.FW * p.FC, Q = (size_t)p.outH * p.outW, HW = (size_t)p.H * p.W;
  for (int i = 0; i < p.groups; ++i) {
    int rc = backward_data_group(s, g, wd, dx + i * p.FC * HW, dxMult, f + i * p.Kg * FV, dy + i * p.Kg * Q, ws, wsBytes, pk, nullptr, nullptr, nullptr);
    if (rc) return rc;
  }
  return MCN_SUCCESS;
}

namespace {
int backward_filter_group(hipStream_t s, const ConvP& p, Wide wd, bool ut, float* df, const float* x, const float* dy,
                          void* ws, size_t wsBytes, ReduceCtx* deferred) {
  WgP q;
  q.xImg = wd.xImg;
  q.dyImg = wd.yImg;
  q.H = p.H; q.W = p.W; q.C = p.C; q.K = p.K;
  q.OH = p.outH; q.OW = p.outW;
  q.FH = p.FH; q.T = p.FH * p.FW;
  q.sy = p.sy; q.sx = p.sx; q.pt = p.pt; q.pl = p.pl; q.dly = p.dy; q.dlx = p.dx;
  q.FV = p.FH * p.FW * p.FC;
  q.M = p.outH * p.outW * p.N;
  {
    // what the product reads of x and dzdy, from the group's first channel on (the uniform-tap test keeps both below
    // 2 GiB; only that variant uses them)
    const long long xb = ((long long)(p.N - 1) * wd.xImg + (long long)p.C * p.H * p.W) * 4;
    const long long yb = ((long long)(p.N - 1) * wd.yImg + (long long)p.K * p.outH * p.outW) * 4;
    q.xBytes = (unsigned)std::min<long long>(xb, 0x7fffffffll);
    q.dyBytes = (unsigned)std::min<long long>(yb, 0x7fffffffll);
  }
  int tiles = 0;
  q.splits = wgrad_splits(p, &tiles);
  const int chunks = (q.M + 31) / 32;
  q.chunkSpan = ((chunks + q.splits - 1) / q.splits) * 32;
  {
    const int BAk = pick_channels_tile(p.K);
    q.byQ = FastDiv(p.outH * p.outW);
    q.byOH = FastDiv(p.outH);
    q.byT = FastDiv(q.T);
    q.byFH = FastDiv(p.FH);
    q.byTiles = FastDiv(tiles);
    q.byTilesK = FastDiv((p.K + BAk - 1) / BAk);
  }
  const size_t nF = (size_t)q.FV * p.K;
  q.byC = FastDiv(p.C);
  float* target = df;
  if (q.splits > 1 || ut) {
    const size_t need = (size_t)q.splits * nF * sizeof(float);
    if (deferred) {
      // the partial banks stay in the caller's buffer until the deferred sum
      target = deferred->base ? (float*)(deferred->base + deferred->offset) : nullptr;
      deferred->offset += align256(need);
      if (deferred->launch && deferred->offset > deferred->capacity)
        return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter: buffer of partial banks too small (%zu < %zu bytes)",
                    deferred->capacity, deferred->offset);
      if (deferred->jobs) {
        ReduceJob j;
        j.df = df; j.partials = target; j.n = nF; j.splits = q.splits; j.tapMajor = ut ? 1 : 0; j.C = p.C; j.T = q.T;
        j.firstBlock = 0; j.blocks = (unsigned)((nF + 63) / 64);
        deferred->jobs->push_back(j);
      }
    } else {
      if (!ws || wsBytes < need)
        return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter: workspace too small (%zu < %zu bytes)", wsBytes, need);
      target = (float*)ws;
    }
  }
  if (deferred && !deferred->launch) return MCN_SUCCESS;
  {
    const unsigned long long ob = (unsigned long long)q.splits * nF * sizeof(float);
    q.outBytes = ob < (1ull << 31) ? (unsigned)ob : 0u;
  }
  const dim3 grid((unsigned)(tiles * q.splits)), block(256);
  const int BA = pick_channels_tile(p.K);
  int rc;
  const bool narrow = pick_rows_tile(p) == 64, wide = pick_rows_tile(p) == 192;
  // Loads straight into LDS wherever the kernel has the form (uniform taps, whole filter tiles), issued a few at a time
  // between the MFMAs: 12-18 % on every layer measured (1x1 layers of ResNet-50 at 32 images 44.3 -> 37.4 us, 3x3x64x64 on
  // 56x56 78.8 -> 67.9 us, 3x3x256x256 on 56x56x256x64 1.95 -> 1.74 ms).  Issued all at once at the top of a step the same
  // loads were a gain only for short launches and a loss for long ones (1.96 -> 2.09 ms).
  const bool direct = ut && p.K % BA == 0;
  if (direct && wide) {
    rc = launch_wgrad<1, 3, 2, 2, true, true>(s, grid, target, x, dy, q);
  } else if (direct && BA == 128) {
    // (128 x 128 tiles with no more workgroups than CUs: three buffers, which leave room for one workgroup on a CU)
    const bool deep = !narrow && (long long)tiles * q.splits <= device_compute_units();
    rc = narrow ? launch_wgrad<2, 1, 2, 2, true, true>(s, grid, target, x, dy, q)
                : (deep ? launch_wgrad<2, 2, 2, 2, true, true, true>(s, grid, target, x, dy, q)
                        : launch_wgrad<2, 2, 2, 2, true, true>(s, grid, target, x, dy, q));
  } else if (direct && BA == 64) {
    rc = narrow ? launch_wgrad<1, 1, 2, 2, true, true>(s, grid, target, x, dy, q) : launch_wgrad<2, 1, 1, 4, true, true>(s, grid, target, x, dy, q);
  } else if (wide) {   // (BA == 64 by pick_rows_tile)
    rc = ut ? launch_wgrad<1, 3, 2, 2, true>(s, grid, target, x, dy, q) : launch_wgrad<1, 3, 2, 2, false>(s, grid, target, x, dy, q);
  } else if (ut) {
    if (BA == 128) rc = narrow ? launch_wgrad<2, 1, 2, 2, true>(s, grid, target, x, dy, q) : launch_wgrad<2, 2, 2, 2, true>(s, grid, target, x, dy, q);
    else if (BA == 64) rc = narrow ? launch_wgrad<1, 1, 2, 2, true>(s, grid, target, x, dy, q) : launch_wgrad<2, 1, 1, 4, true>(s, grid, target, x, dy, q);
    else rc = launch_wgrad<1, 1, 1, 4, true>(s, grid, target, x, dy, q);
  } else {
    if (BA == 128) rc = narrow ? launch_wgrad<2, 1, 2, 2, false>(s, grid, target, x, dy, q) : launch_wgrad<2, 2, 2, 2, false>(s, grid, target, x, dy, q);
    else if (BA == 64) rc = narrow ? launch_wgrad<1, 1, 2, 2, false>(s, grid, target, x, dy, q) : launch_wgrad<2, 1, 1, 4, false>(s, grid, target, x, dy, q);
    else rc = launch_wgrad<1, 1, 1, 4, false>(s, grid, target, x, dy, q);
  }
  if (!rc) rc = check_launch("mcn_conv_backward_filter");
  if (rc || target == df || deferred) return rc;
  KernelTimer timer("conv_wgrad_reduce", s);
  hipLaunchKernelGGL(conv_wgrad_reduce, dim3((unsigned)((nF + 63) / 64)), block, 0, s, df, target, nF, q.splits, ut ? 1 : 0,
                     p.C, q.T);
  return check_launch("mcn_conv_backward_filter(reduce)");
}
}  // namespace

int conv_reduce_batch(hipStream_t s, const ReduceJob* deviceJobs, int nJobs, unsigned totalBlocks) {
  if (nJobs <= 0 || totalBlocks == 0) return MCN_SUCCESS;
  KernelTimer timer("conv_wgrad_reduce_many", s);
  hipLaunchKernelGGL(conv_wgrad_reduce_many, dim3(totalBlocks), dim3(256), 0, s, deviceJobs, nJobs);
  return check_launch("mcn_conv_reduce_batch");
}

int conv_backward_filter_mfma(hipStream_t s, const ConvP& original, float* df, const float* x, const float* dy, void* ws,
                              size_t wsBytes, ReduceCtx* deferred) {
  const ConvP p = fc_view(original);
  const ConvP g = group_view(p);
  const Wide wd = wide_of(p);
  const bool ut = wgrad_uniform_tap(p);
  const size_t FV = (size_t)p.FH * p.FW * p.FC, Q = (size_t)p.outH * p.outW, HW = (size_t)p.H * p.W;
  for (int i = 0; i < p.groups; ++i) {
    int rc = backward_filter_group(s, g, wd, ut, df + i * p.Kg * FV, x + i * p.FC * HW, dy + i * p.Kg * Q, ws, wsBytes, deferred);
    if (rc) return rc;
  }
  return MCN_SUCCESS;
}

}  // namespace mcn
