// Filter gradient (and, from the same pass, bias gradient) of first layers: few input channels, a filter volume of at
// most 160 rows (5x5x3 = 75, 7x7x3 = 147), 32 or 64 filters -- bits/nnconv.cu:230-244,280-311 for such a layer.
//
// The tiled filter-gradient kernel works on 128 x 128 tiles of the bank: a 75 x 32 bank fills 15% of one.  Here
//   * the product dF[k][r] = sum over pixels of dzdy[k][pixel] * patch[r][pixel] runs on v_mfma_f32_32x32x2_f32 with
//     32 filters as the rows of a block, 32 rows of the filter volume as its columns and two pixels per instruction;
//     a wavefront keeps the whole bank (every block of rows x every block of filters) in its accumulators, so an
//     operand read from LDS feeds several instructions and consecutive instructions never wait for each other;
//   * a tile of output pixels (TH rows x TW columns of one image) is staged in LDS by loads that write LDS directly:
//     its dzdy (all filters) and the input pixels its windows read, zero where the window leaves the image (a load past
//     the buffer's end returns zero); a patch row is then "the row's offset inside the window + the pixel's offset
//     inside the tile": one LDS read per operand, no patch matrix anywhere;
//   * the four wavefronts of a workgroup take a quarter of every tile column's pixels each;
//   * a workgroup with several tiles stages tile t + 1 while it multiplies tile t (two buffers; the LDS reads of the
//     product are written as instructions with their own waits, because the compiler would make every LDS access it
//     sees wait for all direct-to-LDS loads in flight, the next tile's included); issuing a tile's loads keeps a
//     wavefront busy for about as long as multiplying it, so several workgroups share a compute unit and one
//     multiplies while another stages;
//   * row R of the volume (the first padded one) reads the constant 1: its column of the product is the sum of dzdy per
//     filter, the bias gradient, for nothing;
//   * workgroups walk the tiles in a fixed order, add their four wavefronts' banks in LDS in wavefront order and leave
//     one partial bank each; a second launch adds the partial banks in workgroup order (deterministic, no atomics).
#include "conv_common.hpp"

#include <algorithm>
#include <atomic>

namespace mcn {
namespace {

typedef __attribute__((address_space(3))) void* first_lds_ptr;


struct FirstP {
  int H, W, Cin, N, FH, FW, K, R;
  int sy, sx, pt, pl, outH, outW;
  int TH, TW;              // output pixels of a tile: TH rows (even) x TW columns, at most 256 in all
  int tilesH, tilesW, tiles;  // tiles per column / per row of tiles / in all (images included)
  int XH, XW;              // input rows and columns a tile's windows read
  int dyPitch;             // floats per filter of the dzdy tile in LDS: whole chunks of 64 pixels, and one float so
                           // that the filters fall into different banks
  int xStepR, xStepC, xStepD;  // 256 elements of the x region on: rows, columns, channels (256 = (D XW + C) XH + R)
  int vec;                 // 16 bytes per lane
  int dyRegion, xRegion;   // floats of the two regions (whole chunks)
  int dyUnits, xChunks;    // dzdy: filters (4 bytes per lane) or chunks of 64 slots (16 bytes); x: chunks of 64 slots
  int XHl, xShift;         // LDS pitch of an x column, and the rows between the aligned first row and the window's
  int XHs;                 // slots per x column (rows, or groups of four rows)
  int TH4, P4;             // 16 bytes per lane: slots per tile column, slots per filter (the pad slot included)
  int dyStepK, dyStepW, dyStepH;  // 256 dzdy slots on = dyStepK filters, dyStepW columns, dyStepH slots
  int bufFloats;           // dzdy region, x region, then 64 floats that start with the constants 0 and 1
  int nbuf;                // 2: the next tile is staged during the product
  int rowChunks;           // chunks of 64 pixels per filter of the dzdy tile
  unsigned dyImgBytes, xImgBytes;  // one image of dzdy and of x
  int nWg;
  int RP;                  // rows of a partial bank: 32 per block of rows
  int wantBias;
  FastDiv byTH, byTH4, byP4, byXHs, byXW, byTilesH, byTilesW, byFH, byFW;
};

__device__ __forceinline__ unsigned first_lds_addr(const float* p) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (unsigned)(size_t)(const __attribute__((address_space(3))) float*)p;
#else
  return 0;
#endif
}

// KB: blocks of 32 filters; RB: blocks of 32 rows of the filter volume (plus the row of ones)
// (wavefronts per SIMD the register budget is set for: the accumulators are 16 KB RB registers)
constexpr int first_waves(int KB, int RB) { return KB * RB >= 8 ? 2 : (KB * RB >= 5 ? 3 : 4); }

template <int KB, int RB>
__global__ __launch_bounds__(256, first_waves(KB, RB)) void conv_first_wgrad(float* __restrict__ partials,
                                                                             const float* __restrict__ x,
                                                                             const float* __restrict__ dy, FirstP p) {
  extern __shared__ float smem[];
  const int T = p.TH * p.TW;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, kh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cw = wave;
  const size_t inPlane = (size_t)p.H * p.W, outPlane = (size_t)p.outH * p.outW;

  // ---- this lane's rows of the filter volume: r = i + FH (j + FW d) reads the window at (i, j) of channel d
  int rOff[RB], bInc[RB], bIncWrap[RB];
  // the wavefront's share of a tile column: pairs of rows q0 ... q0 + nq - 1
  const int halfTH = p.TH / 2, perWave = (halfTH + 3) / 4;
  const int q0 = cw * perWave, nq = max(0, min(q0 + perWave, halfTH) - q0);
  const int nSteps = nq * p.TW;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int r = 32 * rb + l32;
    if (r < p.R) {
      int jd, i, d, j;
      p.byFH.divmod(r, &jd, &i);
      p.byFW.divmod(jd, &d, &j);
      rOff[rb] = p.dyRegion + (d * p.XW + j) * p.XHl + p.xShift + i + (kh + 2 * q0) * p.sy;
      bInc[rb] = 4 * 2 * p.sy;                                          // (bytes) the next pair of rows
      bIncWrap[rb] = 4 * (p.sx * p.XHl - 2 * p.sy * (nq - 1));           // from a column's last pair to the next column
    } else {
      rOff[rb] = p.dyRegion + p.xRegion + ((r == p.R && p.wantBias) ? 1 : 0);
      bInc[rb] = 0;
      bIncWrap[rb] = 0;
    }
  }
  const int aOff = l32 * p.dyPitch + kh + 2 * q0;
  const int aIncWrap = 4 * (p.TH - 2 * (nq - 1));
  if (tid < 2 * p.nbuf) smem[(tid >> 1) * p.bufFloats + p.dyRegion + p.xRegion + (tid & 1)] = (float)(tid & 1);

  // ---- where this lane's slot of the wavefront's first chunks lies (see the staging below)
  int pixW[4], pixH[4];
  unsigned pixRel[4];
  int dk0 = 0, dw0 = 0, dh0 = 0;
  if (p.vec) {
    int j;
    p.byP4.divmod(cw * 64 + lane, &dk0, &j);
    p.byTH4.divmod(j, &dw0, &dh0);
  } else {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      p.byTH.divmod(c * 64 + lane, &pixW[c], &pixH[c]);
      pixRel[c] = 4u * (unsigned)(pixW[c] * p.outH + pixH[c]);
    }
  }

  floatx16 acc[RB][KB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rb][kb][v] = 0.f;

  // (x region: slot = (channel d, column cc, row or group of four rows rr) of the tile's input window)
  int xr0, xc0, xd0;
  {
    int seg;
    p.byXHs.divmod(cw * 64 + lane, &seg, &xr0);
    p.byXW.divmod(seg, &xd0, &xc0);
  }

  // Loads of a tile into a buffer.  Every wavefront issues the same loads for every tile: a lane outside the image,
  // or on a pad slot, reads past the buffer's end instead of sitting out (that gives zero).  Two forms:
  //   * 16 bytes per lane, when the planes' heights and the tile's are multiples of four: a slot is four rows of one
  //     column; dzdy is [filter][slots of the tile, and one pad slot], x is [channel][column][groups of four rows from
  //     the aligned row at or above the window's first]; chunk c of 64 slots is staging wavefront c % 4's;
  //   * 4 bytes per lane otherwise: dzdy by filter (rows cw, cw + 4, ... in chunks of 64 pixels), x by chunks of
  //     64 elements.
  // A lane follows its slot from one of its chunks to the next (256 slots on) by carries, without divisions.
  __amdgpu_buffer_rsrc_t dr, xr;
  unsigned vo[4], so = 0;
  float *dyDst = nullptr, *xT = nullptr;
  int kNext = 0, cNext = 0, row0 = 0, col0 = 0, rr = 0, cc = 0, d = 0, h0 = 0, w0 = 0, dk = 0, dw = 0, dh = 0;
  auto stage_begin = [&](int t, int b) {
    int n, rest, tw, th;
    p.byTilesW.divmod(t, &rest, &tw);   // t = (n tilesH + th) tilesW + tw: tiles of one image together
    p.byTilesH.divmod(rest, &n, &th);
    h0 = th * p.TH;
    w0 = tw * p.TW;
    float* dyT = smem + b * p.bufFloats;
    xT = dyT + p.dyRegion;
    dr = __builtin_amdgcn_make_buffer_rsrc((void*)(dy + (size_t)n * p.K * outPlane), 0, (int)p.dyImgBytes, 0x00020000);
    xr = __builtin_amdgcn_make_buffer_rsrc((void*)(x + (size_t)n * p.Cin * inPlane), 0, (int)p.xImgBytes, 0x00020000);
    if (p.vec) {
      dyDst = dyT + cw * 256;
      dk = dk0;
      dw = dw0;
      dh = dh0;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        vo[c] = (c * 64 + lane < T && h0 + pixH[c] < p.outH && w0 + pixW[c] < p.outW) ? pixRel[c] : 0x80000000u;
      so = 4u * (unsigned)(w0 * p.outH + h0 + cw * (int)outPlane);
      dyDst = dyT + cw * p.dyPitch;
    }
    kNext = cw;
    cNext = cw;
    row0 = h0 * p.sy - p.pt - p.xShift;
    col0 = w0 * p.sx - p.pl;
    rr = xr0;
    cc = xc0;
    d = xd0;
  };
  auto stage_unit = [&]() {
    if (kNext < p.dyUnits) {
      if (p.vec) {
        const bool in = dk < p.K && dw < p.TW && h0 + 4 * dh < p.outH && w0 + dw < p.outW;
        const unsigned off = in ? 4u * (unsigned)(dk * (int)outPlane + (w0 + dw) * p.outH + h0 + 4 * dh) : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)dyDst, 16, (int)off, 0, 0, 0);
        dyDst += 4 * 256;
        // 256 slots on: slot = (dk P4 + dw TH4 + dh), the pad slot of a filter being (dw, dh) = (TW, 0)
        dh += p.dyStepH;
        const int c1 = dh >= p.TH4 ? 1 : 0;
        dh -= c1 ? p.TH4 : 0;
        dw += p.dyStepW + c1;
        dk += p.dyStepK;
        if (dw > p.TW || (dw == p.TW && dh >= 1)) {
          dh -= 1;
          const int c2 = dh < 0 ? 1 : 0;
          dh += c2 ? p.TH4 : 0;
          dw -= p.TW + c2;
          dk += 1;
        }
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)dyDst, 4, (int)vo[0], (int)so, 0, 0);
        if (p.rowChunks > 1) __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)(dyDst + 64), 4, (int)vo[1], (int)so, 0, 0);
        if (p.rowChunks > 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)(dyDst + 128), 4, (int)vo[2], (int)so, 0, 0);
        if (p.rowChunks > 3) __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)(dyDst + 192), 4, (int)vo[3], (int)so, 0, 0);
        so += 16u * (unsigned)outPlane;
        dyDst += 4 * p.dyPitch;
      }
      kNext += 4;
    } else if (cNext < p.xChunks) {
      const int row = row0 + (p.vec ? 4 * rr : rr), col = col0 + cc;
      const bool in = d < p.Cin && (unsigned)row < (unsigned)p.H && (unsigned)col < (unsigned)p.W;
      const unsigned off = in ? 4u * (unsigned)(d * (int)inPlane + col * p.H + row) : 0x80000000u;
      if (p.vec) __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (first_lds_ptr)(xT + cNext * 256), 16, (int)off, 0, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (first_lds_ptr)(xT + cNext * 64), 4, (int)off, 0, 0, 0);
      cNext += 4;
      rr += p.xStepR;
      const int carry = rr >= p.XHs ? 1 : 0;
      rr -= carry ? p.XHs : 0;
      cc += p.xStepC + carry;
      const int wrap = cc >= p.XW ? 1 : 0;
      cc -= wrap ? p.XW : 0;
      d += p.xStepD + wrap;
    }
  };
  auto stage_rest = [&]() {
    while (kNext < p.dyUnits || cNext < p.xChunks) stage_unit();
  };

  // The product over this wavefront's pixels of the tile in buffer b: step s is pair q0 + s % nq of column s / nq.
  // Operands of step s + 1 are read while step s multiplies; a read past the last step repeats the last one.
  auto multiply = [&](int b) {
    if (nSteps == 0) return;
    const unsigned base = first_lds_addr(smem + b * p.bufFloats);
    unsigned aA = base + 4u * (unsigned)aOff;
    unsigned bA[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) bA[rb] = base + 4u * (unsigned)rOff[rb];
    const unsigned kbStride = 4u * 32u * (unsigned)p.dyPitch;
    int issued = 0, qi = 0;
    auto advance = [&]() {
      if (issued + 1 < nSteps) {
        const bool wrap = qi + 1 == nq;
        qi = wrap ? 0 : qi + 1;
        aA += wrap ? (unsigned)aIncWrap : 8u;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) bA[rb] += (unsigned)(wrap ? bIncWrap[rb] : bInc[rb]);
      }
      ++issued;
    };
    auto read = [&](float (&a)[KB], float (&bv)[RB]) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) asm volatile("ds_read_b32 %0, %1" : "=v"(a[kb]) : "v"(aA + kb * kbStride));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) asm volatile("ds_read_b32 %0, %1" : "=v"(bv[rb]) : "v"(bA[rb]));
    };
    auto landed = [&](float (&a)[KB], float (&bv)[RB], bool all) {
      if (all) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(KB + RB) : "memory");
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) asm volatile("" : "+v"(a[kb]));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) asm volatile("" : "+v"(bv[rb]));
    };
    auto mfma = [&](const float (&a)[KB], const float (&bv)[RB]) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) acc[rb][kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kb], bv[rb], acc[rb][kb], 0, 0, 0);
    };
    float a0[KB], b0[RB], a1[KB], b1[RB];
    read(a0, b0);
    for (int s = 0; s < nSteps; s += 2) {
      advance();
      read(a1, b1);
      landed(a0, b0, false);
      mfma(a0, b0);
      advance();
      read(a0, b0);
      landed(a1, b1, false);
      if (s + 1 < nSteps) mfma(a1, b1);
    }
    landed(a0, b0, true);
  };

  auto barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  constexpr int RP = 32 * RB, BANK = 32 * KB * RP;
  int t = blockIdx.x, buf = 0;
  stage_begin(t, 0);
  stage_rest();
  for (; t < p.tiles; t += p.nWg) {
    // tile t has landed (every wavefront's loads), and the other buffer's product is over
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int tn = t + p.nWg;
    if (tn < p.tiles) {
      stage_begin(tn, buf ^ 1);
      stage_rest();
    }
    multiply(buf);
    buf ^= 1;
  }
  barrier();
  // ---- the four wavefronts' banks added in LDS in wavefront order: register v of lane (l32, kh) is filter
  // 8 (v / 4) + 4 kh + v % 4 of its block
  float* mine = smem + (4 * kh) * RP + l32;
  for (int w = 0; w < 4; ++w) {
    if (cw == w) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          float old[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) old[v] = w == 0 ? 0.f : mine[(kb * 32 + 8 * (v / 4) + v % 4) * RP + 32 * rb];
#pragma unroll
          for (int v = 0; v < 16; ++v) mine[(kb * 32 + 8 * (v / 4) + v % 4) * RP + 32 * rb] = old[v] + acc[rb][kb][v];
        }
    }
    barrier();
  }
  // ---- this workgroup's partial bank [filter][row]
  float* out = partials + (size_t)blockIdx.x * BANK;
  for (int i = tid; i < BANK; i += 256) out[i] = smem[i];
}

// dF[r + R k] = sum over the partial banks, in their order (double above the banks' own float sums); row R: the bias
// gradient.  A workgroup: 32 elements of the banks x 32 runs of partial banks, the runs added in order through LDS.
__global__ __launch_bounds__(1024) void conv_first_reduce(float* __restrict__ dF, float* __restrict__ dB,
                                                          const float* __restrict__ partials, int nWg, int K, int R, int RP) {
  __shared__ double part[32][33];
  const int col = threadIdx.x & 31, run = threadIdx.x >> 5;
  const int e = blockIdx.x * 32 + col;
  const int total = K * RP;
  const int per = (nWg + 31) / 32, s0 = run * per, s1 = min(s0 + per, nWg);
  double sum = 0.0;
  if (e < total) {
    const float* src = partials + e;
    int s = s0;
    for (; s + 4 <= s1; s += 4) {
      const float a0 = src[(size_t)s * total], a1 = src[(size_t)(s + 1) * total], a2 = src[(size_t)(s + 2) * total],
                  a3 = src[(size_t)(s + 3) * total];
      sum += (double)a0;
      sum += (double)a1;
      sum += (double)a2;
      sum += (double)a3;
    }
    for (; s < s1; ++s) sum += (double)src[(size_t)s * total];
  }
  part[run][col] = sum;
  __syncthreads();
  if (run == 0 && e < total) {
    double all = 0.0;
#pragma unroll
    for (int i = 0; i < 32; ++i) all += part[i][col];
    const int k = e / RP, r = e - k * RP;
    if (r < R) dF[(size_t)k * R + r] = (float)all;
    else if (r == R && dB) dB[k] = (float)all;
  }
}

bool first_plan(const ConvP& c, FirstP* out, size_t* lds, int* rb, int* kb) {
  if (c.groups != 1 || c.dy != 1 || c.dx != 1 || c.C > 4 || c.C < 1) return false;
  const int R = c.FH * c.FW * c.C;
  if (R + 1 > 160 || (c.K != 32 && c.K != 64)) return false;
  if (c.outH < 2 || c.outW < 1 || c.N < 1) return false;
  if ((size_t)c.K * c.outH * c.outW >= (1u << 29) || (size_t)c.C * c.H * c.W >= (1u << 29)) return false;  // (32-bit byte offsets inside an image)
  FirstP p;
  p.H = c.H; p.W = c.W; p.Cin = c.C; p.N = c.N; p.FH = c.FH; p.FW = c.FW; p.K = c.K; p.R = R;
  p.sy = c.sy; p.sx = c.sx; p.pt = c.pt; p.pl = c.pl; p.outH = c.outH; p.outW = c.outW;
  // 16 bytes per lane when every group of four rows is whole: in the planes and in the tiles
  const int vec = (c.outH % 4 == 0 && c.H % 4 == 0) ? 1 : 0;
  p.vec = vec;
  // tile: whole columns of the output up to 64 rows (even; a multiple of four for 16-byte loads), and some columns:
  // at most 256 pixels, and two buffers for each of the workgroups that share a compute unit (as many as the
  // registers allow wavefronts per SIMD)
  const int unit = vec ? 4 : 2;
  const int wholeH = (c.outH + unit - 1) / unit * unit;
  int TH = std::min(wholeH, 64);
  if (wholeH > 64) {  // cut tall columns into equal parts
    const int parts = (wholeH + 63) / 64;
    TH = ((wholeH + parts - 1) / parts + unit - 1) / unit * unit;
  }
  const int shift = vec ? ((c.pt % 4) == 0 ? 0 : 4 - c.pt % 4) : 0;  // (the window's first row is -pad plus a multiple of four)
  const int XH = (TH - 1) * c.sy + c.FH;
  const int XHl = vec ? (shift + XH + 3) / 4 * 4 : XH;
  int TW = std::max(1, std::min(c.outW, 256 / TH));
  auto dy_floats = [&](int tw) {
    const int T = TH * tw;
    return vec ? ((size_t)c.K * (T / 4 + 1) + 63) / 64 * 256 : ((size_t)c.K * ((T + 63) / 64 * 64 + 1) + 63) / 64 * 64;
  };
  auto x_floats = [&](int tw) {
    const size_t XW = (size_t)(tw - 1) * c.sx + c.FW;
    return vec ? ((size_t)c.C * XW * (XHl / 4) + 63) / 64 * 256 : ((size_t)c.C * XW * XH + 63) / 64 * 64;
  };
  auto floats = [&](int tw) { return dy_floats(tw) + x_floats(tw) + 64; };
  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  const int cap = tunable("conv_first_max_wg", 0);  // (tests: a few workgroups walk many tiles of a small input)
  const int tilesH = (c.outH + TH - 1) / TH;
  auto widest = [&](size_t budget) {
    int tw = std::max(1, std::min(c.outW, 256 / TH));
    while (tw > 1 && floats(tw) * sizeof(float) > budget) --tw;
    return tw;
  };
  // Either every tile gets a workgroup of its own and the chip holds them all at once (tiles up to 38 KB), or the
  // workgroups walk the tiles with two buffers each, as many per compute unit as the registers allow wavefronts per SIMD
  bool walk = true;
  {
    TW = widest(38 * 1024);
    const size_t one = std::max((size_t)c.K * 32 * ((R + 1 + 31) / 32) * sizeof(float), floats(TW) * sizeof(float));
    const long long tiles = (long long)tilesH * ((c.outW + TW - 1) / TW) * c.N;
    const long long atOnce = cap > 0 ? cap : (long long)cus * std::min<size_t>(4, (160 * 1024) / (one + 1024));
    if (floats(TW) * sizeof(float) <= 38 * 1024 && tiles <= atOnce) walk = false;
  }
  const int perCu = first_waves(c.K / 32, (R + 1 + 31) / 32);
  if (walk) {
    const size_t budget = (160 * 1024 / perCu - 1024) / 2;
    TW = widest(budget);
    if (floats(TW) * sizeof(float) > budget) return false;
  }
  if (vec && (TH * c.sy) % 4 != 0) return false;  // (cannot be: TH is a multiple of four)
  p.TH = TH; p.TW = TW;
  p.tilesH = (c.outH + TH - 1) / TH;
  p.tilesW = (c.outW + TW - 1) / TW;
  const long long tiles = (long long)p.tilesH * p.tilesW * c.N;
  if (tiles >= (1ll << 30)) return false;
  p.tiles = (int)tiles;
  p.XH = XH;
  p.XW = (TW - 1) * c.sx + c.FW;
  p.XHl = XHl;
  p.xShift = shift;
  p.XHs = vec ? XHl / 4 : XH;
  p.xStepR = 256 % p.XHs;
  p.xStepC = (256 / p.XHs) % p.XW;
  p.xStepD = (256 / p.XHs) / p.XW;
  p.TH4 = std::max(1, TH / 4);
  p.P4 = TH * TW / 4 + 1;
  p.dyPitch = vec ? 4 * p.P4 : (TH * TW + 63) / 64 * 64 + 1;
  p.dyRegion = (int)dy_floats(TW);
  p.xRegion = (int)x_floats(TW);
  p.xChunks = vec ? p.xRegion / 256 : p.xRegion / 64;
  p.dyUnits = vec ? p.dyRegion / 256 : c.K;
  {
    const int dj = 256 % p.P4;
    p.dyStepK = 256 / p.P4;
    p.dyStepW = dj / p.TH4;
    p.dyStepH = dj % p.TH4;
  }
  p.bufFloats = (int)floats(TW);
  p.rowChunks = (TH * TW + 63) / 64;
  p.dyImgBytes = (unsigned)((size_t)c.K * c.outH * c.outW * 4);
  p.xImgBytes = (unsigned)((size_t)c.C * c.H * c.W * 4);
  *rb = (R + 1 + 31) / 32;
  *kb = c.K / 32;
  p.RP = 32 * *rb;
  // (the bank the workgroup's last sums make uses the same LDS)
  const size_t bank = (size_t)c.K * p.RP * sizeof(float);
  p.nbuf = walk ? 2 : 1;
  p.nWg = (int)std::min<long long>(tiles, walk ? (cap > 0 ? cap : (long long)perCu * cus) : tiles);
  *lds = std::max(bank, (size_t)p.nbuf * p.bufFloats * sizeof(float));
  p.wantBias = 0;
  p.byTH = FastDiv(TH); p.byTH4 = FastDiv(p.TH4); p.byP4 = FastDiv(p.P4); p.byXHs = FastDiv(p.XHs); p.byXW = FastDiv(p.XW);
  p.byTilesH = FastDiv(p.tilesH); p.byTilesW = FastDiv(p.tilesW);
  p.byFH = FastDiv(c.FH); p.byFW = FastDiv(c.FW);
  *out = p;
  return true;
}

template <int KB, int RB>
int first_launch(hipStream_t s, size_t lds, float* partials, const float* x, const float* dy, const FirstP& p) {
  static std::atomic<size_t> raised[kMaxDevices];
  const int dev = current_device();
  if (lds > 64 * 1024 && (dev < 0 || dev >= kMaxDevices || lds > raised[dev].load(std::memory_order_acquire))) {
    if (hipFuncSetAttribute((const void*)conv_first_wgrad<KB, RB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return fail(MCN_UNSUPPORTED, "mcn_conv_backward_filter: %zu bytes of LDS refused", lds);
    }
    if (dev >= 0 && dev < kMaxDevices) raised[dev].store(lds, std::memory_order_release);
  }
  hipLaunchKernelGGL((conv_first_wgrad<KB, RB>), dim3((unsigned)p.nWg), dim3(256), lds, s, partials, x, dy, p);
  return MCN_SUCCESS;
}

}  // namespace

// ------------------------------------------------------------------------------------------------------------------
// Input gradient of a first layer (stride 1): dzdx has at most four channels, so the product is short of matrix
// shape in one direction (bits/nnconv.cu:247-277 for such a layer).  Here it runs on vector FMAs from LDS:
//   * a workgroup takes a tile of input pixels of one image (whole columns up to 64 rows x a few columns) and stages
//     the dzdy its windows reach, every filter's plane, by loads that write LDS directly (zero outside the image);
//   * a lane owns two vertically adjacent pixels and all channels: for a filter and a window column it reads FH + 1
//     consecutive rows of dzdy from LDS (8-byte reads) and uses each for both pixels -- 2 FH C multiply-adds per
//     (FH + 1) / 2 reads; the weights are wave-uniform, read as scalars;
//   * the four wavefronts take a quarter of the filters each; their sums are added in wavefront order through LDS.
namespace {

struct FirstD {
  int H, W, N, FW, K, pt, pl, outH, outW;
  int TH, TW;               // input pixels of a tile
  int halfTH, cols;         // lanes: pair of rows u = lane % halfTH of column lane / halfTH (cols columns per tile)
  int LH, LW;               // rows and columns of dzdy a tile reaches: TH + FH - 1, TW + FW - 1
  int kPer;                 // filters per wavefront
  int tilesH, tilesW, tiles;
  int chunks;               // chunks of 64 floats of the staged region [filter][column][row]
  int stepR, stepC, stepK;  // 256 slots on = stepK filters, stepC columns, stepR rows
  unsigned dyImgBytes;
  FastDiv byLH, byLW, byTilesH, byTilesW, byHalfTH, byTH, byTW;
};

template <int FH, int FW, int C>
__global__ __launch_bounds__(256) void conv_first_dgrad(float* __restrict__ dx, const float* __restrict__ f,
                                                        const float* __restrict__ dy, FirstD p) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const size_t inPlane = (size_t)p.H * p.W, outPlane = (size_t)p.outH * p.outW;
  int n, rest, tw, th;
  p.byTilesW.divmod((int)blockIdx.x, &rest, &tw);
  p.byTilesH.divmod(rest, &n, &th);
  const int h0 = th * p.TH, w0 = tw * p.TW;

  // ---- dzdy of the tile: slot (filter k, column cc, row rr) is output pixel (h0 + pt - (FH - 1) + rr,
  // w0 + pl - (FW - 1) + cc); a lane follows its slot from chunk to chunk (256 slots on) by carries
  {
    const __amdgpu_buffer_rsrc_t dr =
        __builtin_amdgcn_make_buffer_rsrc((void*)(dy + (size_t)n * p.K * outPlane), 0, (int)p.dyImgBytes, 0x00020000);
    int seg, rr, k, cc;
    p.byLH.divmod(wave * 64 + lane, &seg, &rr);
    p.byLW.divmod(seg, &k, &cc);
    const int oh0 = h0 + p.pt - (FH - 1), ow0 = w0 + p.pl - (FW - 1);
    for (int c = wave; c < p.chunks; c += 4) {
      const int oh = oh0 + rr, ow = ow0 + cc;
      const bool in = k < p.K && (unsigned)oh < (unsigned)p.outH && (unsigned)ow < (unsigned)p.outW;
      const unsigned off = in ? 4u * (unsigned)(k * (int)outPlane + ow * p.outH + oh) : 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (first_lds_ptr)(smem + c * 64), 4, (int)off, 0, 0, 0);
      rr += p.stepR;
      const int carry = rr >= p.LH ? 1 : 0;
      rr -= carry ? p.LH : 0;
      cc += p.stepC + carry;
      const int wrap = cc >= p.LW ? 1 : 0;
      cc -= wrap ? p.LW : 0;
      k += p.stepK + wrap;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- this lane's two pixels: rows h0 + 2 u, h0 + 2 u + 1 of column w0 + col
  int col, u;
  p.byHalfTH.divmod(lane, &col, &u);
  const int colR = min(col, p.TW - 1);  // (lanes past the tile's columns read a column that exists and write nothing)
  float acc[2][C];
#pragma unroll
  for (int c = 0; c < C; ++c) acc[0][c] = acc[1][c] = 0.f;
  const int kEnd = min(p.K, (wave + 1) * p.kPer);
  for (int k = wave * p.kPer; k < kEnd; ++k) {
    // (the window's columns unrolled: the scalar loads of the weights and the LDS reads of all of them are in flight
    // before the first multiply)
#pragma unroll
    for (int j = 0; j < FW; ++j) {
      // rows 2 u ... 2 u + FH of column colR + FW - 1 - j: the window rows both pixels reach through column tap j
      const float2* src = (const float2*)(smem + (k * p.LW + colR + FW - 1 - j) * p.LH + 2 * u);
      float v[FH + 1];
#pragma unroll
      for (int e = 0; e < (FH + 1) / 2; ++e) {
        const float2 pair = src[e];
        v[2 * e] = pair.x;
        v[2 * e + 1] = pair.y;
      }
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const float* wv = f + (size_t)FH * (j + FW * (c + C * k));
#pragma unroll
        for (int i = 0; i < FH; ++i) {
          const float w = wv[i];
          acc[0][c] = fmaf(v[FH - 1 - i], w, acc[0][c]);
          acc[1][c] = fmaf(v[FH - i], w, acc[1][c]);
        }
      }
    }
  }
  __syncthreads();
  // ---- the four wavefronts' sums: [wavefront][channel][column][row], added in wavefront order
  const int T = p.TH * p.TW;
  if (col < p.TW) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
      float* dst = smem + (wave * C + c) * T + col * p.TH + 2 * u;
      dst[0] = acc[0][c];
      dst[1] = acc[1][c];
    }
  }
  __syncthreads();
  float* dxImg = dx + (size_t)n * C * inPlane;
  for (int i = tid; i < C * T; i += 256) {
    const float sum = ((smem[i] + smem[C * T + i]) + smem[2 * C * T + i]) + smem[3 * C * T + i];
    int seg, row, c, cw;
    p.byTH.divmod(i, &seg, &row);
    p.byTW.divmod(seg, &c, &cw);
    const int ih = h0 + row, iw = w0 + cw;
    if (ih < p.H && iw < p.W) dxImg[(size_t)c * inPlane + (size_t)iw * p.H + ih] = sum;
  }
}

bool first_data_plan(const ConvP& c, FirstD* out, size_t* lds) {
  if (c.groups != 1 || c.dy != 1 || c.dx != 1 || c.sy != 1 || c.sx != 1 || c.C > 4 || c.C < 1) return false;
  if ((c.FH != 3 && c.FH != 5 && c.FH != 7) || c.FW != c.FH) return false;  // (square windows: both loops over them are unrolled)
  if (c.K < 4 || c.N < 1 || c.H < 2 || c.outH < 1 || c.outW < 1 || tunable("conv_no_first", 0)) return false;
  if ((size_t)c.K * c.outH * c.outW >= (1u << 29) || (size_t)c.C * c.H * c.W >= (1u << 29)) return false;
  FirstD p;
  p.H = c.H; p.W = c.W; p.N = c.N; p.FW = c.FW; p.K = c.K; p.pt = c.pt; p.pl = c.pl; p.outH = c.outH; p.outW = c.outW;
  const int evenH = (c.H + 1) & ~1;
  int TH = std::min(evenH, 64);
  if (evenH > 64) {
    const int parts = (evenH + 63) / 64;
    TH = (((evenH + parts - 1) / parts) + 1) & ~1;
  }
  p.TH = TH;
  p.halfTH = TH / 2;
  p.cols = 64 / p.halfTH;
  p.TW = std::min(p.cols, c.W);
  p.LH = TH + c.FH - 1;
  p.LW = p.TW + c.FW - 1;
  p.kPer = (c.K + 3) / 4;
  const size_t region = ((size_t)c.K * p.LW * p.LH + 63) / 64 * 64;
  const size_t sums = (size_t)4 * c.C * TH * p.TW;
  const size_t bytes = std::max(region, sums) * sizeof(float);
  if (bytes > 64 * 1024) return false;
  p.chunks = (int)(region / 64);
  p.stepR = 256 % p.LH;
  p.stepC = (256 / p.LH) % p.LW;
  p.stepK = (256 / p.LH) / p.LW;
  p.tilesH = (c.H + TH - 1) / TH;
  p.tilesW = (c.W + p.TW - 1) / p.TW;
  const long long tiles = (long long)p.tilesH * p.tilesW * c.N;
  if (tiles >= (1ll << 30)) return false;
  p.tiles = (int)tiles;
  p.dyImgBytes = (unsigned)((size_t)c.K * c.outH * c.outW * 4);
  p.byLH = FastDiv(p.LH); p.byLW = FastDiv(p.LW); p.byTilesH = FastDiv(p.tilesH); p.byTilesW = FastDiv(p.tilesW);
  p.byHalfTH = FastDiv(p.halfTH); p.byTH = FastDiv(TH); p.byTW = FastDiv(p.TW);
  *out = p;
  *lds = bytes;
  return true;
}

template <int FH>
void first_data_launch(hipStream_t s, int C, size_t lds, float* dx, const float* f, const float* dy, const FirstD& p) {
  const dim3 grid((unsigned)p.tiles), block(256);
  switch (C) {
    case 1: hipLaunchKernelGGL((conv_first_dgrad<FH, FH, 1>), grid, block, lds, s, dx, f, dy, p); break;
    case 2: hipLaunchKernelGGL((conv_first_dgrad<FH, FH, 2>), grid, block, lds, s, dx, f, dy, p); break;
    case 3: hipLaunchKernelGGL((conv_first_dgrad<FH, FH, 3>), grid, block, lds, s, dx, f, dy, p); break;
    default: hipLaunchKernelGGL((conv_first_dgrad<FH, FH, 4>), grid, block, lds, s, dx, f, dy, p); break;
  }
}

}  // namespace

bool conv_first_backward_data_supported(const ConvP& c) {
  FirstD p;
  size_t lds;
  return first_data_plan(c, &p, &lds);
}

// dzdx of a first layer with stride 1 (nothing is accumulated onto it)
int conv_first_backward_data(hipStream_t s, const ConvP& c, float* dx, const float* f, const float* dy) {
  FirstD p;
  size_t lds;
  if (!first_data_plan(c, &p, &lds)) return fail(MCN_UNSUPPORTED, "mcn_conv_backward_data: not a first layer");
  KernelTimer timer("conv_first_dgrad", s);
  if (c.FH == 3) first_data_launch<3>(s, c.C, lds, dx, f, dy, p);
  else if (c.FH == 5) first_data_launch<5>(s, c.C, lds, dx, f, dy, p);
  else first_data_launch<7>(s, c.C, lds, dx, f, dy, p);
  return check_launch("mcn_conv_backward_data");
}

bool conv_first_backward_filter_supported(const ConvP& c) {
  FirstP p;
  size_t lds;
  int rb, kb;
  if (c.C > 4) return false;  // (the common answer, before any look-up)
  return !tunable("conv_no_first", 0) && first_plan(c, &p, &lds, &rb, &kb);
}

size_t conv_first_workspace_bytes(const ConvP& c) {
  FirstP p;
  size_t lds;
  int rb, kb;
  if (!first_plan(c, &p, &lds, &rb, &kb)) return 0;
  return (size_t)p.nWg * p.K * p.RP * sizeof(float);
}

// dF (and dB when not null) of a first layer.  ws: conv_first_workspace_bytes.
int conv_first_backward_filter(hipStream_t s, const ConvP& c, float* dF, float* dB, const float* x, const float* dy, void* ws,
                               size_t wsBytes) {
  FirstP p;
  size_t lds;
  int rb, kb;
  if (!first_plan(c, &p, &lds, &rb, &kb)) return fail(MCN_UNSUPPORTED, "mcn_conv_backward_filter: not a first layer");
  const int banks = p.nWg;
  const size_t need = (size_t)banks * p.K * p.RP * sizeof(float);
  if (!ws || wsBytes < need) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter: workspace too small (%zu < %zu bytes)", wsBytes, need);
  p.wantBias = dB ? 1 : 0;
  float* partials = (float*)ws;
  int rc = MCN_SUCCESS;
  {
    KernelTimer timer("conv_first_wgrad", s);
    if (kb == 1) {
      switch (rb) {
        case 1: rc = first_launch<1, 1>(s, lds, partials, x, dy, p); break;
        case 2: rc = first_launch<1, 2>(s, lds, partials, x, dy, p); break;
        case 3: rc = first_launch<1, 3>(s, lds, partials, x, dy, p); break;
        case 4: rc = first_launch<1, 4>(s, lds, partials, x, dy, p); break;
        default: rc = first_launch<1, 5>(s, lds, partials, x, dy, p); break;
      }
    } else {
      switch (rb) {
        case 1: rc = first_launch<2, 1>(s, lds, partials, x, dy, p); break;
        case 2: rc = first_launch<2, 2>(s, lds, partials, x, dy, p); break;
        case 3: rc = first_launch<2, 3>(s, lds, partials, x, dy, p); break;
        case 4: rc = first_launch<2, 4>(s, lds, partials, x, dy, p); break;
        default: rc = first_launch<2, 5>(s, lds, partials, x, dy, p); break;
      }
    }
  }
  if (rc) return rc;
  rc = check_launch("mcn_conv_backward_filter");
  if (rc) return rc;
  KernelTimer timer("conv_first_reduce", s);
  hipLaunchKernelGGL(conv_first_reduce, dim3((unsigned)((p.K * p.RP + 31) / 32)), dim3(1024), 0, s, dF, dB, partials, banks, p.K,
                     p.R, p.RP);
  return check_launch("mcn_conv_backward_filter");
}

}  // namespace mcn
