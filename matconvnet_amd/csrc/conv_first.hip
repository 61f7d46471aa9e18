// Kernels for first layers (one to four input channels, 32 or 64 filters): the filter gradient with the bias gradient
// from the same pass (this comment), the input gradient at stride 1 and the forward product (further down, each with
// a comment of its own).
//
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

// ------------------------------------------------------------------------------------------------------------------
// Forward product of a first layer (bits/nnconv.cu:126-161 for such a layer): y[k][pixel] = sum over the rows r of the
// filter volume of w[k][r] patch[r][pixel] + b[k], on v_mfma_f32_32x32x2_f32 with 32 filters as rows, 32 output pixels
// as columns and two rows of the volume per instruction.
//   * A workgroup keeps the whole bank in LDS, [row][filter] (staged once), and walks tiles of TH x TW output pixels of
//     one image; a tile's input pixels are staged as in the filter-gradient kernel above (direct-to-LDS loads, zero
//     outside the image), and a patch element is again "offset of the row inside the window + offset of the pixel
//     inside the tile": one LDS read per operand.
//   * Its four wavefronts are WK groups of 32 filters x WP groups of pixel blocks; a wavefront holds up to eight blocks
//     of 32 pixels in its accumulators (started at the bias), so a weight read from LDS feeds up to eight instructions.
//   * The tile of x is small next to the arithmetic it feeds (every staged pixel meets all filters), so one buffer and
//     the compiler's own waits are enough here: the loads of a tile are a tenth of its matrix instructions.
namespace {

struct FirstF {
  int H, W, Cin, N, FH, FW, K, R;
  int sy, sx, pt, pl, outH, outW;
  int TH, TW, T;
  int tilesH, tilesW, tiles, nWg;
  int XW, XHl, xShift, XHs;   // columns of x a tile reads; LDS pitch of a column; rows before the window's first; slots per column
  int vec;                    // 16 bytes per lane
  int xChunks;                // chunks of 64 slots of the x region
  int steps;                  // pairs of rows of the filter volume
  int WP, bpw;                // pixel groups of wavefronts; blocks of 32 pixels per wavefront
  int xStepR, xStepC, xStepD;
  unsigned xImgBytes;
  int wFloats, tabFloats;     // floats of the bank in LDS and of the row table (whole chunks of 64)
  FastDiv byXHs, byXW, byTilesH, byTilesW, byTH, byRows, byFH, byFW;
};

// BPW: blocks of 32 pixels per wavefront (a constant, so that a step's LDS reads are issued together, ahead of its
// matrix instructions)
template <int BPW>
__global__ __launch_bounds__(256, 2) void conv_first_fwd(float* __restrict__ y, const float* __restrict__ x,
                                                         const float* __restrict__ f, const float* __restrict__ bias, FirstF p) {
  extern __shared__ float smem[];
  const int KP = p.K + 1;                             // (pitch of a row of the bank: staging writes it down the columns)
  float* wT = smem;                                   // [2 steps + 2][K + 1]: rows past the volume's last are zero
  int* rowTab = (int*)(smem + p.wFloats);             // [2 steps + 4]: offset of a row of the volume inside a pixel's window
  float* xT = smem + p.wFloats + p.tabFloats;         // [channel][column][row]
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, kh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wp = wave % p.WP, wk = wave / p.WP;
  const size_t inPlane = (size_t)p.H * p.W, outPlane = (size_t)p.outH * p.outW;

  // the bank: read along the rows of a filter (consecutive addresses for consecutive threads), twenty loads in flight
  // per thread; written transposed
  {
    const int rows = 2 * p.steps + 2, total = rows * p.K;
    for (int base = tid; base < total; base += 20 * 256) {
      float v[20];
      int at[20];
#pragma unroll
      for (int u = 0; u < 20; ++u) {
        const int idx = base + u * 256;
        int k, r;
        p.byRows.divmod(min(idx, total - 1), &k, &r);
        at[u] = idx < total ? r * KP + k : -1;
        v[u] = (idx < total && r < p.R) ? f[(size_t)r + (size_t)p.R * k] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 20; ++u)
        if (at[u] >= 0) wT[at[u]] = v[u];
    }
  }
  for (int r = tid; r < 2 * p.steps + 4; r += 256) {
    int jd, i, d, j;
    p.byFH.divmod(r, &jd, &i);   // r = i + FH (j + FW d)
    p.byFW.divmod(jd, &d, &j);
    rowTab[r] = r < p.R ? p.xShift + (d * p.XW + j) * p.XHl + i : 0;
  }
  // this lane's pixels: block wp + WP j of the tile, pixel 32 block + l32 = (column w, row h) of the tile
  int pixOff[BPW], pixWH[BPW];
#pragma unroll
  for (int j = 0; j < BPW; ++j) {
    const int pix = min(32 * (wp + p.WP * j) + l32, p.T - 1);
    int w, h;
    p.byTH.divmod(pix, &w, &h);
    pixOff[j] = w * p.sx * p.XHl + h * p.sy;
    pixWH[j] = (32 * (wp + p.WP * j) + l32 < p.T) ? (w | (h << 16)) : 0x7fff7fff;  // (past the tile: never inside the output)
  }
  float bv[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) bv[v] = bias ? bias[wk * 32 + 8 * (v / 4) + 4 * kh + v % 4] : 0.f;
  int xr0, xc0, xd0;
  {
    int seg;
    p.byXHs.divmod(wave * 64 + lane, &seg, &xr0);
    p.byXW.divmod(seg, &xd0, &xc0);
  }

  for (int t = blockIdx.x; t < p.tiles; t += p.nWg) {
    int n, rest, tw, th;
    p.byTilesW.divmod(t, &rest, &tw);
    p.byTilesH.divmod(rest, &n, &th);
    const int h0 = th * p.TH, w0 = tw * p.TW;
    __syncthreads();  // (the tile before this one has been multiplied; the first time: the bank is in place)
    {
      const __amdgpu_buffer_rsrc_t xr =
          __builtin_amdgcn_make_buffer_rsrc((void*)(x + (size_t)n * p.Cin * inPlane), 0, (int)p.xImgBytes, 0x00020000);
      const int row0 = h0 * p.sy - p.pt - p.xShift, col0 = w0 * p.sx - p.pl;
      int rr = xr0, cc = xc0, d = xd0;
      for (int c = wave; c < p.xChunks; c += 4) {
        const int row = row0 + (p.vec ? 4 * rr : rr), col = col0 + cc;
        const bool in = d < p.Cin && (unsigned)row < (unsigned)p.H && (unsigned)col < (unsigned)p.W;
        const unsigned off = in ? 4u * (unsigned)(d * (int)inPlane + col * p.H + row) : 0x80000000u;
        if (p.vec) __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (first_lds_ptr)(xT + c * 256), 16, (int)off, 0, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (first_lds_ptr)(xT + c * 64), 4, (int)off, 0, 0, 0);
        rr += p.xStepR;
        const int carry = rr >= p.XHs ? 1 : 0;
        rr -= carry ? p.XHs : 0;
        cc += p.xStepC + carry;
        const int wrap = cc >= p.XW ? 1 : 0;
        cc -= wrap ? p.XW : 0;
        d += p.xStepD + wrap;
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    floatx16 acc[BPW];
#pragma unroll
    for (int j = 0; j < BPW; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][v] = bv[v];
    // rows 2 s + kh of the volume, s = 0, 1, ...; the operands of step s + 1 are read while step s multiplies (the
    // row's offset inside the window comes from a table, read two steps ahead)
    const float* aPtr = wT + kh * KP + wk * 32 + l32;
    float aNext = aPtr[0];
    float bNext[BPW];
    {
      const int off = rowTab[kh];
#pragma unroll
      for (int j = 0; j < BPW; ++j) bNext[j] = xT[off + pixOff[j]];
    }
    int offAfter = rowTab[2 + kh];
    for (int s = 0; s < p.steps; ++s) {
      const float a = aNext;
      float b[BPW];
#pragma unroll
      for (int j = 0; j < BPW; ++j) b[j] = bNext[j];
      // (past the last step: the table and the bank have two more rows, of zeros)
      aNext = aPtr[2 * (s + 1) * KP];
#pragma unroll
      for (int j = 0; j < BPW; ++j) bNext[j] = xT[offAfter + pixOff[j]];
      offAfter = rowTab[2 * (s + 2) + kh];
      if (s == p.steps - 1 && (p.R & 1)) {
        // the row past an odd volume's last: its weight is zero, and so must its patch be (x may hold infinities)
#pragma unroll
        for (int j = 0; j < BPW; ++j) b[j] = kh ? 0.f : b[j];
      }
#pragma unroll
      for (int j = 0; j < BPW; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[j], acc[j], 0, 0, 0);
    }
    // register v of lane (l32, kh) of block j: filter wk 32 + 8 (v / 4) + 4 kh + v % 4, the lane's pixel of the block
    float* yImg = y + (size_t)n * p.K * outPlane;
#pragma unroll
    for (int j = 0; j < BPW; ++j) {
      const int ow = w0 + (pixWH[j] & 0xffff), oh = h0 + (pixWH[j] >> 16);
      if (ow < p.outW && oh < p.outH) {
        float* dst = yImg + (size_t)ow * p.outH + oh;
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(size_t)(wk * 32 + 8 * (v / 4) + 4 * kh + v % 4) * outPlane] = acc[j][v];
      }
    }
  }
}

bool first_fwd_plan(const ConvP& c, FirstF* out, size_t* lds) {
  if (c.groups != 1 || c.dy != 1 || c.dx != 1 || c.C > 4 || c.C < 1 || c.FH < 2) return false;
  const int R = c.FH * c.FW * c.C;
  // (small volumes are all output: 3x3x3x64 on 224x224x3x32 writes 411 MB for 5.5 GFLOP, and the general kernel's
  // stores are the better ones: 152 against 162 us)
  if (R < 48 || R + 1 > 160 || (c.K != 32 && c.K != 64) || tunable("conv_no_first", 0)) return false;
  if (c.outH < 1 || c.outW < 1 || c.N < 1) return false;
  if ((size_t)c.K * c.outH * c.outW >= (1u << 29) || (size_t)c.C * c.H * c.W >= (1u << 29)) return false;
  FirstF p;
  p.H = c.H; p.W = c.W; p.Cin = c.C; p.N = c.N; p.FH = c.FH; p.FW = c.FW; p.K = c.K; p.R = R;
  p.sy = c.sy; p.sx = c.sx; p.pt = c.pt; p.pl = c.pl; p.outH = c.outH; p.outW = c.outW;
  p.steps = (R + 1) / 2;
  p.vec = c.H % 4 == 0 ? 1 : 0;  // (whole groups of four rows are inside the image or outside)
  const int WK = c.K / 32;
  p.WP = 4 / WK;
  // rows of a tile: whole columns up to 64 rows, in equal parts (a multiple of four rows when x is staged 16 bytes
  // per lane: the window's first row must keep its place inside a group of four from tile to tile)
  const int unit = p.vec ? 4 : 1;
  int TH = (std::min(c.outH, 64) + unit - 1) / unit * unit;
  if (c.outH > 64) {
    const int parts = (c.outH + 63) / 64;
    TH = ((c.outH + parts - 1) / parts + unit - 1) / unit * unit;
  }
  const int shift = p.vec ? ((c.pt % 4) == 0 ? 0 : 4 - c.pt % 4) : 0;
  const int XH = (TH - 1) * c.sy + c.FH;
  const int XHl = p.vec ? (shift + XH + 3) / 4 * 4 : XH;
  p.tabFloats = (2 * p.steps + 4 + 63) / 64 * 64;
  p.wFloats = ((2 * p.steps + 2) * (c.K + 1) + 63) / 64 * 64;
  const size_t wFloats = (size_t)p.wFloats + p.tabFloats;
  auto x_floats = [&](int tw) {
    const size_t XW = (size_t)(tw - 1) * c.sx + c.FW;
    return p.vec ? ((size_t)c.C * XW * (XHl / 4) + 63) / 64 * 256 : ((size_t)c.C * XW * XH + 63) / 64 * 64;
  };
  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  const int perCu = 2;  // (one workgroup per compute unit: 122 against 105 us on a ResNet stem)
  const size_t budget = 160 * 1024 / perCu - 1024;
  // columns of a tile: among those that fit (LDS; eight blocks of 32 pixels per wavefront), the width with the
  // shortest longest walk -- tiles per workgroup x blocks per wavefront, and half a block's time per tile besides
  const int tilesH = (c.outH + TH - 1) / TH;
  long long best = -1;
  int TW = 0;
  for (int tw = std::min(c.outW, 32 * 8 * p.WP / TH); tw >= 1; --tw) {
    if ((wFloats + x_floats(tw)) * sizeof(float) > budget) continue;
    const long long tiles = (long long)tilesH * ((c.outW + tw - 1) / tw) * c.N;
    const long long nWg = std::min<long long>(tiles, (long long)cus * perCu);
    const int blocks = (TH * tw + 31) / 32, bpw = (blocks + p.WP - 1) / p.WP;
    const long long cost = ((tiles + nWg - 1) / nWg) * (2 * bpw + 1);
    if (best < 0 || cost < best) {
      best = cost;
      TW = tw;
    }
  }
  if (TW < 1) return false;
  p.TH = TH; p.TW = TW; p.T = TH * TW;
  p.bpw = ((p.T + 31) / 32 + p.WP - 1) / p.WP;
  if (p.bpw > 8) return false;
  p.tilesH = tilesH;
  p.tilesW = (c.outW + TW - 1) / TW;
  const long long tiles = (long long)p.tilesH * p.tilesW * c.N;
  if (tiles >= (1ll << 30)) return false;
  p.tiles = (int)tiles;
  p.nWg = (int)std::min<long long>(tiles, (long long)cus * perCu);
  p.XW = (TW - 1) * c.sx + c.FW;
  p.XHl = XHl;
  p.xShift = shift;
  p.XHs = p.vec ? XHl / 4 : XH;
  p.xChunks = (int)(x_floats(TW) / (p.vec ? 256 : 64));
  p.xStepR = 256 % p.XHs;
  p.xStepC = (256 / p.XHs) % p.XW;
  p.xStepD = (256 / p.XHs) / p.XW;
  p.xImgBytes = (unsigned)((size_t)c.C * c.H * c.W * 4);
  p.byXHs = FastDiv(p.XHs); p.byXW = FastDiv(p.XW); p.byTilesH = FastDiv(p.tilesH); p.byTilesW = FastDiv(p.tilesW);
  p.byTH = FastDiv(TH); p.byRows = FastDiv(2 * p.steps + 2); p.byFH = FastDiv(c.FH); p.byFW = FastDiv(c.FW);
  *lds = (wFloats + x_floats(TW)) * sizeof(float);
  *out = p;
  return true;
}

}  // namespace

bool conv_first_forward_supported(const ConvP& c) {
  if (c.C > 4) return false;
  FirstF p;
  size_t lds;
  return first_fwd_plan(c, &p, &lds);
}

// y = conv(x, f) + bias of a first layer (nothing is accumulated onto y)
int conv_first_forward(hipStream_t s, const ConvP& c, float* y, const float* x, const float* f, const float* bias) {
  FirstF p;
  size_t lds;
  if (!first_fwd_plan(c, &p, &lds)) return fail(MCN_UNSUPPORTED, "mcn_conv_forward: not a first layer");
  typedef void (*Kernel)(float*, const float*, const float*, const float*, FirstF);
  static const Kernel kernels[8] = {conv_first_fwd<1>, conv_first_fwd<2>, conv_first_fwd<3>, conv_first_fwd<4>,
                                    conv_first_fwd<5>, conv_first_fwd<6>, conv_first_fwd<7>, conv_first_fwd<8>};
  const Kernel kernel = kernels[p.bpw - 1];
  static std::atomic<size_t> raised[kMaxDevices][8];
  const int dev = current_device();
  if (lds > 64 * 1024 && (dev < 0 || dev >= kMaxDevices || lds > raised[dev][p.bpw - 1].load(std::memory_order_acquire))) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return fail(MCN_UNSUPPORTED, "mcn_conv_forward: %zu bytes of LDS refused", lds);
    }
    if (dev >= 0 && dev < kMaxDevices) raised[dev][p.bpw - 1].store(lds, std::memory_order_release);
  }
  KernelTimer timer("conv_first_fwd", s);
  hipLaunchKernelGGL(kernel, dim3((unsigned)p.nWg), dim3(256), lds, s, y, x, f, bias, p);
  return check_launch("mcn_conv_forward");
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
