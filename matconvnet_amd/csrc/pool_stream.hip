// Max-pooling backward, streaming form (the fast path for planes whose columns are whole 16-byte cells: heights that
// are a multiple of 4 in single precision, of 2 in double).
//
// Same arithmetic and visiting order as the ordered-pass kernel of pool.hip -- one accumulator of the data type per
// input element, every output adds its dzdy to the first maximum of its window, outputs reach an accumulator in
// ascending (output column, output row) order (bits/nnpooling.cu:33-66,190-206) -- organised so that HBM
// never waits for the arithmetic:
//   * persistent workgroups: workgroup b of G takes tiles b, b + G, ... (a tile = all rows of TW columns of one
//     plane) and loads its NEXT tile's x and dzdy into registers before it works on the current one;
//   * the x columns a tile's windows read live in LDS inside a -inf frame whose image rows start on a
//     16-byte boundary, so staging is one 16-byte LDS write per 16-byte global load and windows need no
//     clipping tests;
//   * the winner search is straight-line compare/select code (no divergent branches), the rank tables are
//     packed into two scalars;
//   * accumulators are streamed out with non-temporal 16-byte stores and reset by the thread that read them.
// No atomics; bit-identical to the CPU loops.
#include "mcn_internal.hpp"

#include <algorithm>
#include <atomic>

#pragma clang fp contract(off)

namespace mcn {
namespace {

// A 16-byte cell of the data type: four floats or two doubles.
template <typename E> struct Cell;
template <> struct Cell<float> {
  typedef float vec __attribute__((ext_vector_type(4)));
  static constexpr int n = 4;
};
template <> struct Cell<double> {
  typedef double vec __attribute__((ext_vector_type(2)));
  static constexpr int n = 2;
};

struct PoolS {
  int H, W, outH, outW, sy, sx, pt, pl, poolH, poolW;
  int H4;        // cells per column: H / (elements per cell)
  int top;       // frame row of image row 0: the padding rounded up to whole cells
  int Hp;        // frame pitch in elements (whole cells)
  int maxC;      // widest frame over the tiles of a plane, in columns
  int TW, tilesPerPlane, totalTiles;
  int accumulate;
  int walk;  // 0: tiles dealt round-robin to workgroups; 1: one contiguous run each; 2: round-robin inside each XCD's eighth;
             // 3: planes dealt round-robin to XCDs, a plane's tiles round-robin to that XCD's workgroups
  int KH, nPasses;
  unsigned rankHpk, rankWpk;  // 4 bits per window offset: (pool - 1 - offset) / stride
  FastDiv byTiles, bySx, byOutH, byH4, byBorder;  // byBorder: border rows per frame column (Hp - H)
  int outStepQ, outStepR;    // threads per workgroup = outStepQ * outH + outStepR
  int cellStepQ, cellStepR;  // threads per workgroup = cellStepQ * H4 + cellStepR
};

// Uniform description of one tile: all rows of the image columns [w0, w0 + nW) of one plane.
template <typename E>
struct Tile {
  int w0, nW;          // owned columns
  int owLo, nOut;      // first output column whose window touches the tile; outputs touching it
  int cLo, nC;         // frame column 0 is image column cLo (may be negative: padding); frame columns
  int ca;              // first image column present in the frame
  int nCells;          // 16-byte cells of x to load: columns [ca, cb) x H/4
  const E* xsrc;       // x at (row 0, column ca)
  const E* dsrc;       // dzdy at (row 0, column owLo)
  E* out;              // dzdx at (row 0, column w0)
};

template <typename E>
__device__ __forceinline__ Tile<E> tile_geometry(const PoolS& p, int tile, int poolW, const E* xPlane, const E* dyPlane,
                                                 E* dxPlane) {
  Tile<E> g;
  g.w0 = tile * p.TW;
  const int w1 = min(g.w0 + p.TW, p.W);
  g.nW = w1 - g.w0;
  const int loNum = g.w0 + p.pl - poolW + 1;
  g.owLo = loNum <= 0 ? 0 : p.bySx.div(loNum + p.sx - 1);
  const int owHi = min(p.outW - 1, p.bySx.div(w1 - 1 + p.pl));
  const int nOW = max(owHi - g.owLo + 1, 0);
  g.nOut = nOW * p.outH;
  g.cLo = g.owLo * p.sx - p.pl;
  g.nC = nOW > 0 ? (nOW - 1) * p.sx + poolW : 0;
  g.ca = max(g.cLo, 0);
  const int cb = min(g.cLo + g.nC, p.W);
  g.nCells = max(cb - g.ca, 0) * p.H4;
  g.xsrc = xPlane + g.ca * p.H;
  g.dsrc = dyPlane + g.owLo * p.outH;
  g.out = dxPlane + g.w0 * p.H;
  return g;
}

// Issues the global loads of tile g: this thread's cells of x and its outputs' dzdy.
template <typename E, int OPT, int XPT, int T>
__device__ __forceinline__ void prefetch_tile(typename Cell<E>::vec (&xr)[XPT], E (&dr)[OPT], const Tile<E>& g, int tid) {
  // Lanes past the end re-read the last element instead of being masked off (their copies are never used):
  // a clamped index costs one instruction, a masked region four.
  if (g.nCells > 0) {
#pragma unroll
    for (int u = 0; u < XPT; ++u) xr[u] = ((const typename Cell<E>::vec*)g.xsrc)[min(tid + T * u, g.nCells - 1)];
  }
  if (g.nOut > 0) {
#pragma unroll
    for (int k = 0; k < OPT; ++k) dr[k] = g.dsrc[min(tid + T * k, g.nOut - 1)];
  }
}

// max(a, b) as the hardware instruction: returns the other operand when one is NaN.  (The library call would
// add an instruction per operand to quieten signalling NaNs, which plays no role here.)
__device__ __forceinline__ float hw_max(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ double hw_max(double a, double b) {
  double r;
  asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// a finished cell of accumulators on its way out: written once, not read again by this launch
template <typename V>
__device__ __forceinline__ void stream_store_cell(V* p, const V v) {
#if MCN_NT_STORE
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

// LDS-only barrier: waits for this wave's LDS traffic, not for the global loads of the next tile in flight
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// OPT outputs and XPT 16-byte cells of x per thread and tile; NP > 0: the number of passes, known at compile time.
// T threads per workgroup.
template <typename E, int PH, int PW, int NP, int OPT, int XPT, int T>
__global__ __launch_bounds__(T) void pool_max_backward_stream(E* __restrict__ dx, const E* __restrict__ x,
                                                                const E* __restrict__ dy, PoolS p) {
  typedef typename Cell<E>::vec vec;
  constexpr int VE = Cell<E>::n;
  const E minusInf = -(E)INFINITY;
  const vec zeroCell = (vec)(E)0;
  extern __shared__ __align__(16) unsigned char smemBytes[];
  E* acc = (E*)smemBytes;        // [TW * H] accumulators, all +0 between tiles
  E* frame = acc + p.TW * p.H;   // [maxC * Hp] x inside its -inf frame; frame row r = image row r - top
  // after the frame: one 16-byte cell that swallows the staging writes of idle lanes, and one element per lane
  // that swallows the additions of lanes sitting out a pass
  const int trashCell = p.maxC * p.Hp;                      // relative to frame
  const int idleAcc = p.TW * p.H + p.maxC * p.Hp + VE + threadIdx.x;  // relative to acc
  const int tid = threadIdx.x;
  const int poolH = PH > 0 ? PH : p.poolH, poolW = PW > 0 ? PW : p.poolW;

  // Tiles are dealt so that the workgroups running at any moment cover one contiguous stretch of each tensor
  // (DRAM rows are used up while they are open) and so that the tiles of one plane, which read each other's border
  // columns, sit behind one L2 (walk 3: planes round-robin over the XCDs, a plane's tiles round-robin over that XCD's
  // workgroups).  Measured on the 112x112x64x32 3x3/2 case, cold caches: walk 3 fetches 128.6 MB per launch through the
  // fabric (the tensors' 128.5 MB once) in 44 us; walk 0 (tiles round-robin over all workgroups) 153.5 MB in the same
  // 44 us, 46.5 us when each XCD walks its own eighth of the tiles that way, 50 us when every workgroup owns one
  // contiguous run of tiles.
  const int G = (int)gridDim.x;
  int t0, t1, step, zFirst = 0, zStep = 1;
  if (p.walk == 0) {
    t0 = blockIdx.x;
    t1 = p.totalTiles;
    step = G;
  } else if (p.walk == 1) {
    const int lb = xcd_contiguous_id(blockIdx.x, G);
    t0 = (int)(((long long)lb * p.totalTiles) / G);
    t1 = (int)(((long long)(lb + 1) * p.totalTiles) / G);
    step = 1;
  } else if (p.walk == 2) {
    const int nx = min(kNumXcd, G);  // groups of workgroups; with 8 or more workgroups, one group per XCD
    const int xcd = blockIdx.x % nx, j = blockIdx.x / nx;
    step = G / nx + (xcd < G % nx ? 1 : 0);
    t0 = (int)(((long long)xcd * p.totalTiles) / nx) + j;
    t1 = (int)(((long long)(xcd + 1) * p.totalTiles) / nx);
  } else {
    // planes dealt round-robin to the XCDs (hardware deals workgroup b to XCD b mod 8): the tiles of one plane, which
    // share their halo columns, meet in one L2, and the chip as a whole still covers one contiguous stretch.
    // Here t counts the tiles of this XCD's planes zFirst, zFirst + zStep, ...
    zStep = min(kNumXcd, G);
    zFirst = blockIdx.x % zStep;
    const int j = blockIdx.x / zStep;
    const int planes = p.byTiles.div(p.totalTiles);
    step = G / zStep + (zFirst < G % zStep ? 1 : 0);
    t0 = j;
    t1 = zFirst < planes ? ((planes - zFirst + zStep - 1) / zStep) * p.tilesPerPlane : 0;
  }
  if (t0 >= t1) return;

  // ---- once: accumulators at +0; the frame rows above and below the image at -inf (no tile writes them)
  for (int i = tid; i < p.TW * p.H4; i += T) ((vec*)acc)[i] = zeroCell;
  {
    const int nb = p.Hp - p.H;
    for (int i = tid; i < p.maxC * nb; i += T) {
      int c, k;
      p.byBorder.divmod(i, &c, &k);
      frame[c * p.Hp + (k < p.top ? k : k + p.H)] = minusInf;
    }
  }

  // ---- per-thread constants that no tile changes
  // outputs o = tid + T k of a tile: tile-relative output column oCol, output row oRow
  int oRow[OPT], oCol[OPT], orgOff[OPT], locBase[OPT];
  {
    int owr, oh;
    p.byOutH.divmod(tid, &owr, &oh);
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      oRow[k] = oh;
      oCol[k] = owr;
      orgOff[k] = owr * p.sx * p.Hp + oh * p.sy + p.top - p.pt;  // window origin inside the frame
      locBase[k] = owr * p.sx * p.H + oh * p.sy - p.pt;           // its accumulator, before the tile's column shift
      owr += p.outStepQ;
      oh += p.outStepR;
      if (oh >= p.outH) {
        oh -= p.outH;
        ++owr;
      }
    }
  }
  // cells i = tid + T u of the tile's x: column i / H4 after the first present one, rows VE (i % H4) ...
  int cellDst[XPT];  // frame position when the first present column is frame column 0
  {
    int c, s;
    p.byH4.divmod(tid, &c, &s);
#pragma unroll
    for (int u = 0; u < XPT; ++u) {
      cellDst[u] = c * p.Hp + p.top + VE * s;
      c += p.cellStepQ;
      s += p.cellStepR;
      if (s >= p.H4) {
        s -= p.H4;
        ++c;
      }
    }
  }

  // ---- walk the tiles t0, t0 + step, ... < t1
  const size_t planeIn = (size_t)p.H * p.W, planeOut = (size_t)p.outH * p.outW;
  vec xr[XPT];  // native vectors: these stay in registers under conditional assignment
  E dr[OPT];
  Tile<E> cur;
  {
    int z, tile;
    p.byTiles.divmod(t0, &z, &tile);
    z = zFirst + zStep * z;
    cur = tile_geometry(p, tile, poolW, x + z * planeIn, dy + z * planeOut, dx + z * planeIn);
  }
  prefetch_tile<E, OPT, XPT, T>(xr, dr, cur, tid);

  // The accumulators of a finished tile are written to memory at the start of the next iteration, so their
  // stores have a whole tile's worth of work to complete before this wave next waits on its memory counter.
  E* prevOut = dx;
  int prevIn4 = 0;

  for (int t = t0; t < t1; t += step) {
    const int nIn4 = cur.nW * p.H4;
    // Everything this wave has in flight (this tile's loads, the previous tile's stores) is needed or long
    // done by now.  Waiting here, outside any branch, also tells the compiler that nothing is pending on any
    // path, so it places no memory waits of its own in the arithmetic below.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    // ---- registers -> LDS (image cells only; the -inf rows above and below are permanent)
    {
      const int colShift = (cur.ca - cur.cLo) * p.Hp;
#pragma unroll
      for (int u = 0; u < XPT; ++u)
        *(vec*)(frame + (tid + T * u < cur.nCells ? cellDst[u] + colShift : trashCell)) = xr[u];
      // frame columns left / right of the image (first and last tiles of a plane only)
      if (cur.cLo < 0)
        for (int r = tid; r < colShift; r += T) frame[r] = minusInf;
      const int c0 = p.W - cur.cLo;
      if (cur.nC > c0)
        for (int r = tid; r < (cur.nC - c0) * p.Hp; r += T) frame[c0 * p.Hp + r] = minusInf;
    }
    E dv[OPT];
#pragma unroll
    for (int k = 0; k < OPT; ++k) dv[k] = dr[k];
    // ---- previous tile: stream its accumulators out, leaving +0 (or this tile's derInput when accumulating)
    for (int i = tid; i < prevIn4; i += T) {
      const vec a = ((const vec*)acc)[i];
      ((vec*)acc)[i] = zeroCell;
      stream_store_cell((vec*)prevOut + i, a);
    }
    if (p.accumulate)
      for (int i = tid; i < nIn4; i += T) ((vec*)acc)[i] = ((const vec*)cur.out)[i];
    lds_barrier();

    // ---- next tile's loads go out now and land while this tile is computed
    Tile<E> nxt = cur;
    if (t + step < t1) {
      int z, tile;
      p.byTiles.divmod(t + step, &z, &tile);
      z = zFirst + zStep * z;
      nxt = tile_geometry(p, tile, poolW, x + z * planeIn, dy + z * planeOut, dx + z * planeIn);
      prefetch_tile<E, OPT, XPT, T>(xr, dr, nxt, tid);
    }

    // ---- winner of each owned output: first maximum of its window, scanning column by column
    E best[OPT];
    int code[OPT];  // 8 * column offset + row offset of the winner, -1 when nothing beats -inf
    const E* org[OPT];
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      org[k] = frame + (tid + T * k < cur.nOut ? orgOff[k] : 0);  // idle lanes read a valid window
      best[k] = minusInf;
      code[k] = -1;
    }
    if (PH > 0 && PW > 0) {
      E v[OPT][PW > 0 ? PW : 1][PH > 0 ? PH : 1];
#pragma unroll
      for (int k = 0; k < OPT; ++k)
#pragma unroll
        for (int j = 0; j < PW; ++j)
#pragma unroll
          for (int i = 0; i < PH; ++i) v[k][j][i] = org[k][j * p.Hp + i];
      // the OPT compare/select chains advance together, so no chain waits on its own previous compare
#pragma unroll
      for (int j = 0; j < PW; ++j)
#pragma unroll
        for (int i = 0; i < PH; ++i)
#pragma unroll
          for (int k = 0; k < OPT; ++k) {
            code[k] = v[k][j][i] > best[k] ? (8 * j + i) : code[k];
            best[k] = hw_max(best[k], v[k][j][i]);
          }
    } else {
      for (int j = 0; j < poolW; ++j)
        for (int i = 0; i < poolH; ++i)
#pragma unroll
          for (int k = 0; k < OPT; ++k) {
            const E v = org[k][j * p.Hp + i];
            code[k] = v > best[k] ? (8 * j + i) : code[k];
            best[k] = hw_max(best[k], v);
          }
    }
    // ---- the winner's accumulator and the output's rank among the outputs sharing that winner
    int loc[OPT], rank[OPT];
    const int shift = cur.cLo - cur.w0;  // frame column 0 relative to the tile's first column
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      const int bj = code[k] >> 3, bi = code[k] & 7;
      const int w = oCol[k] * p.sx + bj + shift;  // tile-relative column of the winner
      const bool ok = code[k] >= 0 && tid + T * k < cur.nOut && (unsigned)w < (unsigned)cur.nW;
      const int ra = (int)((p.rankHpk >> (4 * bi)) & 15u), rb = (int)((p.rankWpk >> (4 * bj)) & 15u);
      rank[k] = (min(cur.owLo + oCol[k], rb) * p.KH + min(oRow[k], ra)) | (ok ? 0 : -1);  // -1: routes nothing
      loc[k] = locBase[k] + (shift + bj) * p.H + bi;
    }

    // ---- ordered passes: in pass r the outputs of rank r add into their winner's accumulator
    // (a lane sitting out a pass adds into its private idle slot: a select instead of a masked region)
    if (NP > 0) {
#pragma unroll
      for (int r = 0; r < NP; ++r) {
        E a[OPT];
        int at[OPT];
#pragma unroll
        for (int k = 0; k < OPT; ++k) {
          at[k] = rank[k] == r ? loc[k] : idleAcc;
          a[k] = acc[at[k]];
        }
        // (outputs of equal rank never share a winner, so the real addresses of one pass are all distinct)
#pragma unroll
        for (int k = 0; k < OPT; ++k) acc[at[k]] = a[k] + dv[k];
        lds_barrier();
      }
    } else {
      for (int r = 0; r < p.nPasses; ++r) {
#pragma unroll
        for (int k = 0; k < OPT; ++k)
          if (rank[k] == r) acc[loc[k]] = acc[loc[k]] + dv[k];
        lds_barrier();
      }
    }
    prevOut = cur.out;
    prevIn4 = nIn4;
    cur = nxt;
  }
  // ---- last tile
  for (int i = tid; i < prevIn4; i += T) stream_store_cell((vec*)prevOut + i, ((const vec*)acc)[i]);
}

// One instantiation: opts it into more than 64 KB of LDS when the tile needs that (once per device), then launches.
template <typename E, int PH, int PW, int NP, int OPT, int XPT, int T>
bool launch_stream(hipStream_t s, dim3 grid, size_t lds, E* dx, const E* x, const E* dy, const PoolS& p) {
  static std::atomic<size_t> raised[kMaxDevices];
  const int dev = current_device();
  if (lds > 64 * 1024 && (dev < 0 || dev >= kMaxDevices || lds > raised[dev].load(std::memory_order_acquire))) {
    if (hipFuncSetAttribute((const void*)pool_max_backward_stream<E, PH, PW, NP, OPT, XPT, T>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    if (dev >= 0 && dev < kMaxDevices) raised[dev].store(lds, std::memory_order_release);
  }
  KernelTimer timer("pool_backward_stream", s);
  hipLaunchKernelGGL((pool_max_backward_stream<E, PH, PW, NP, OPT, XPT, T>), grid, dim3((unsigned)T), lds, s, dx, x, dy, p);
  return true;
}

// Launches the streaming kernel when the problem fits it.  Returns true when the work was enqueued.
template <typename E>
bool stream_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, E* derInput, const E* x,
                   const E* derOutput, int accumulate) {
  constexpr int VE = Cell<E>::n;
  if (g->H % VE != 0 || !aligned16(derInput) || !aligned16(x)) return false;
  if (g->poolH > 8 || g->poolW > 8) return false;
  const int kh = (g->poolH + g->strideY - 1) / g->strideY, kw = (g->poolW + g->strideX - 1) / g->strideX;
  if (kh * kw > 4) return false;  // windows overlapping more than 2 x 2 outputs: the ordered-pass kernel of pool.hip is faster
  if (tunable("pool_force_gather", 0)) return false;
  const size_t planes = (size_t)g->C * g->N;

  PoolS p;
  p.H = g->H; p.W = g->W; p.outH = outH; p.outW = outW;
  p.sy = g->strideY; p.sx = g->strideX; p.pt = g->padTop; p.pl = g->padLeft;
  p.poolH = g->poolH; p.poolW = g->poolW;
  p.H4 = g->H / VE;
  p.top = (g->padTop + VE - 1) & ~(VE - 1);
  const int rows = std::max(p.top + g->H, p.top - g->padTop + (outH - 1) * g->strideY + g->poolH);
  p.Hp = (rows + VE - 1) & ~(VE - 1);
  p.accumulate = accumulate ? 1 : 0;
  p.walk = 3;
  p.KH = kh;
  p.nPasses = kh * kw;
  p.rankHpk = p.rankWpk = 0;
  for (int i = 0; i < g->poolH; ++i) p.rankHpk |= (unsigned)((g->poolH - 1 - i) / g->strideY) << (4 * i);
  for (int i = 0; i < g->poolW; ++i) p.rankWpk |= (unsigned)((g->poolW - 1 - i) / g->strideX) << (4 * i);

  // widest tile whose LDS fits the budget and whose outputs and cells fit 4 per thread
  const int threads = 256;  // (512 and 1024 threads measured no faster on 3x3 / 2 windows)
  // (the budget is for single precision; double precision takes the same tiles in twice the bytes)
  const size_t slotBytes = (VE + (size_t)threads) * sizeof(E), scale = sizeof(E) / sizeof(float);
  const size_t budget =
      std::min<size_t>(std::max(tunable("pool_lds_bytes", 16 * 1024), 1024) * scale, 150 * 1024) - slotBytes;
  int TW = 0, maxOut = 0, maxCells = 0, maxC = 0;
  size_t lds = 0;
  for (int nT = 1; nT <= p.W; ++nT) {
    const int cand = (p.W + nT - 1) / nT;
    if (nT > 1 && cand == (p.W + nT - 2) / (nT - 1)) continue;
    int worstOut = 0, worstCells = 0, worstC = 0;
    for (int w0 = 0; w0 < p.W; w0 += cand) {
      const int w1 = std::min(w0 + cand, p.W);
      const int num = w0 + p.pl - p.poolW + 1;
      const int owLo = num <= 0 ? 0 : (num + p.sx - 1) / p.sx;
      const int owHi = std::min(p.outW - 1, (w1 - 1 + p.pl) / p.sx);
      const int nOW = std::max(owHi - owLo + 1, 0);
      const int cLo = owLo * p.sx - p.pl, nC = nOW > 0 ? (nOW - 1) * p.sx + p.poolW : 0;
      const int ca = std::max(cLo, 0), cb = std::min(cLo + nC, p.W);
      worstOut = std::max(worstOut, nOW * p.outH);
      worstCells = std::max(worstCells, std::max(cb - ca, 0) * p.H4);
      worstC = std::max(worstC, nC);
    }
    worstC = std::max(worstC, p.poolW);  // idle lanes read the window at the frame origin
    const size_t need = ((size_t)cand * p.H + (size_t)worstC * p.Hp) * sizeof(E);
    if (need <= budget && worstOut <= 4 * threads && worstCells <= 4 * threads) {
      TW = cand;
      maxOut = worstOut;
      maxCells = worstCells;
      maxC = worstC;
      lds = need;
      break;
    }
  }
  if (TW == 0) return false;
  const size_t tilesPerPlane = (size_t)(p.W + TW - 1) / TW;
  if (planes * tilesPerPlane >= (1ull << 31)) return false;
  p.TW = TW;
  p.maxC = maxC;
  p.tilesPerPlane = (int)tilesPerPlane;
  p.totalTiles = (int)(planes * tilesPerPlane);
  p.byTiles = FastDiv((int)tilesPerPlane);
  p.bySx = FastDiv(p.sx);
  p.byOutH = FastDiv(p.outH);
  p.byH4 = FastDiv(p.H4);
  p.byBorder = FastDiv(std::max(p.Hp - p.H, 1));
  p.outStepQ = threads / p.outH;
  p.outStepR = threads % p.outH;
  p.cellStepQ = threads / p.H4;
  p.cellStepR = threads % p.H4;
  const int opt = std::max((maxOut + threads - 1) / threads, 1), xpt = std::max((maxCells + threads - 1) / threads, 1);
  lds += slotBytes;  // the idle-lane cell and slots

  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  const int perCu = std::min(3, (int)std::max<size_t>((160 * 1024) / std::max<size_t>(lds, 1), 1));
  const int blocks = (int)std::min<long long>(p.totalTiles, (long long)cus * perCu);
  const dim3 grid((unsigned)blocks);
  bool launched = true;
#define MCN_POOL_STREAM_T(PHF, PWF, NPF, OPTF, XPTF, TF) \
  launched = launch_stream<E, PHF, PWF, NPF, OPTF, XPTF, TF>(s, grid, lds, derInput, x, derOutput, p)
#define MCN_POOL_STREAM(PHF, PWF, NPF, OPTF, XPTF) MCN_POOL_STREAM_T(PHF, PWF, NPF, OPTF, XPTF, 256)
#define MCN_POOL_STREAM_XPT(PHF, PWF, NPF, OPTF)               \
  do {                                                         \
    if (xpt == 1) MCN_POOL_STREAM(PHF, PWF, NPF, OPTF, 1);      \
    else if (xpt == 2) MCN_POOL_STREAM(PHF, PWF, NPF, OPTF, 2); \
    else if (xpt == 3) MCN_POOL_STREAM(PHF, PWF, NPF, OPTF, 3); \
    else MCN_POOL_STREAM(PHF, PWF, NPF, OPTF, 4);               \
  } while (0)
#define MCN_POOL_STREAM_OPT(PHF, PWF, NPF)                   \
  do {                                                       \
    if (opt == 1) MCN_POOL_STREAM_XPT(PHF, PWF, NPF, 1);      \
    else if (opt == 2) MCN_POOL_STREAM_XPT(PHF, PWF, NPF, 2); \
    else if (opt == 3) MCN_POOL_STREAM_XPT(PHF, PWF, NPF, 3); \
    else MCN_POOL_STREAM_XPT(PHF, PWF, NPF, 4);               \
  } while (0)
  // the common shapes get their window and pass count at compile time
  if (p.poolH == 3 && p.poolW == 3 && p.nPasses == 4) MCN_POOL_STREAM_OPT(3, 3, 4);        // 3x3, stride 2
  else if (p.poolH == 2 && p.poolW == 2 && p.nPasses == 1) MCN_POOL_STREAM_OPT(2, 2, 1);   // 2x2, stride 2
  else if (p.poolH == 3 && p.poolW == 3) MCN_POOL_STREAM_OPT(3, 3, 0);
  else if (p.poolH == 2 && p.poolW == 2) MCN_POOL_STREAM_OPT(2, 2, 0);
  else MCN_POOL_STREAM_OPT(0, 0, 0);
#undef MCN_POOL_STREAM_OPT
#undef MCN_POOL_STREAM_XPT
#undef MCN_POOL_STREAM
#undef MCN_POOL_STREAM_T
  return launched;
}

}  // namespace

bool pool_max_backward_stream_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, float* derInput,
                                     const float* x, const float* derOutput, int accumulate) {
  return stream_launch<float>(s, g, outH, outW, derInput, x, derOutput, accumulate);
}
bool pool_max_backward_stream_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, double* derInput,
                                     const double* x, const double* derOutput, int accumulate) {
  return stream_launch<double>(s, g, outH, outW, derInput, x, derOutput, accumulate);
}

}  // namespace mcn
