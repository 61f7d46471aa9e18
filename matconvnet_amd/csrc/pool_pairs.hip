// Max-pooling backward for 3x3 windows at stride 2 with one row and one column of padding in front, planes whose
// height is a multiple of 4: the down-sampling layer of residual networks (112x112 -> 56x56).
//
// Same result, bit for bit, as the CPU loops of the reference (bits/nnpooling.cu:33-66,170-214): every output adds its
// dzdy to the first maximum of its window, and the additions into one element happen in ascending (output column,
// output row) order.  Organised so that the memory stream never waits for the arithmetic:
//   * persistent workgroups walk tiles (a tile = all rows of 2L columns of one plane).  The x columns a tile's windows
//     read and the tile's dzdy are contiguous in memory; they are copied into LDS by buffer loads whose destination is
//     LDS (16 bytes per lane, no registers, no LDS write instructions), into three rotating stages, so two tiles are
//     in flight while a third is worked on;
//   * stage A (one thread per 16-byte cell of an output-column pair): the winners of the two windows whose centre
//     rows lie in the cell -- first element strictly greater than everything before it, column by column from -inf,
//     NaN never wins -- written with their dzdy to a table in LDS;
//   * stage B (same thread, one tile later): the eight dzdx elements of the cell's two columns are sums, started at
//     +0, over the (at most six) windows that reach them, taken from the table in the reference's order, in
//     registers, and go straight to memory with non-temporal 16-byte stores.  No accumulators in LDS, no atomics.
//   * stage A of tile k+1 and stage B of tile k share one barrier interval: one barrier per tile.
// Rows and columns in front of the image are read as copies of row / column 0: a copy scanned before its original can
// only win in its place, so the winner is moved back onto the original afterwards.
#include "mcn_internal.hpp"

#include <algorithm>
#include <atomic>

#pragma clang fp contract(off)

namespace mcn {
namespace {

constexpr int kChunk = 1024;  // bytes one wavefront's 16-byte-per-lane load moves

struct PairP {
  int H, W, outH, outW, H4;
  int L;                // output columns (= pairs of dzdx columns) per tile
  int tilesPerPlane;
  int planes, nx;       // nx: XCDs the planes are dealt to (8, or 1 for fewer than 8 planes)
  int stages;           // 2 or 3 rotating stages of a tile's x and dzdy in LDS
  int perCu;            // workgroups that share a compute unit and its pool of tiles (1: every workgroup on its own)
  int share[9];         // member j of a group takes share[j+1] - share[j] of every 64 tiles of the pool (share[0] = 0)
  int tpitch;           // table entries per output column (outH + 2: the last two never win)
  int xChunks, dyChunks;  // 1 KB chunks of a stage that hold x / dzdy
  unsigned xBytes, dyBytes;
  FastDiv byH4, byTiles;
};

__host__ __device__ __forceinline__ float bits_float(int v) { return __builtin_bit_cast(float, v); }
__host__ __device__ __forceinline__ int float_bits(float v) { return __builtin_bit_cast(int, v); }

struct PairTile {
  int z, a;        // plane, first output column
  int nPairs;      // output columns of this tile: min(L, outW - a)
  int shift;       // 1 when the tile starts at the image's left edge (its first window's first column is padding)
  unsigned xOff, dyOff;  // byte offsets of the tile's first x column / first dzdy column
  size_t outOff;   // float offset of dzdx column 2a
};

__host__ __device__ __forceinline__ PairTile pair_tile(const PairP& p, int xcd, int t) {
  PairTile g;
  int zi, ti;
  p.byTiles.divmod(t, &zi, &ti);
  g.z = xcd + p.nx * zi;
  g.a = ti * p.L;
  g.nPairs = min(p.L, p.outW - g.a);
  g.shift = g.a == 0 ? 1 : 0;
  const int cLo = max(2 * g.a - 1, 0);
  g.xOff = (unsigned)(((size_t)g.z * p.H * p.W + (size_t)cLo * p.H) * 4);
  g.dyOff = (unsigned)(((size_t)g.z * p.outH * p.outW + (size_t)g.a * p.outH) * 4);
  g.outOff = (size_t)g.z * p.H * p.W + (size_t)(2 * g.a) * p.H;
  return g;
}

__host__ __device__ __forceinline__ float pair_max(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
  float r;  // the hardware instruction returns the other operand when one is NaN
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
#else
  return b > a ? b : a;  // (host instantiation: CPU checks of the indexing)
#endif
}

// LDS accesses of the two stages.  On the device they are written as instructions: the compiler cannot tell which LDS
// bytes a buffer load with an LDS destination fills, so it makes every LDS access it sees wait for ALL such loads in
// flight, the next two tiles' included -- the loop would run one tile at a time.  The kernel's own wait (one counted
// s_waitcnt per tile, before the barrier) is what orders these reads behind the loads that filled them.
#if defined(__HIP_DEVICE_COMPILE__)
typedef float pair_v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned lds_addr(const float* p) {
  return (unsigned)(size_t)(const __attribute__((address_space(3))) float*)p;
}
#endif

// rows 4s ... 4s+3 (m) and the row before them (up) of three columns, and two dzdy values
__host__ __device__ __forceinline__ void pair_read_a(float4 (&m)[3], float (&up)[3], float2& d, const float* c0,
                                                     const float* c1, const float* c2, int upOff, const float* dp) {
#if defined(__HIP_DEVICE_COMPILE__)
  v4f m0, m1, m2;
  float u0, u1, u2;
  pair_v2f dd;
  asm volatile(
      "ds_read_b128 %0, %7\n\t"
      "ds_read_b128 %1, %8\n\t"
      "ds_read_b128 %2, %9\n\t"
      "ds_read_b32 %3, %10\n\t"
      "ds_read_b32 %4, %11\n\t"
      "ds_read_b32 %5, %12\n\t"
      "ds_read_b64 %6, %13\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(m0), "=&v"(m1), "=&v"(m2), "=&v"(u0), "=&v"(u1), "=&v"(u2), "=&v"(dd)
      : "v"(lds_addr(c0)), "v"(lds_addr(c1)), "v"(lds_addr(c2)), "v"(lds_addr(c0 + upOff)), "v"(lds_addr(c1 + upOff)),
        "v"(lds_addr(c2 + upOff)), "v"(lds_addr(dp))
      : "memory");
  m[0] = make_float4(m0.x, m0.y, m0.z, m0.w);
  m[1] = make_float4(m1.x, m1.y, m1.z, m1.w);
  m[2] = make_float4(m2.x, m2.y, m2.z, m2.w);
  up[0] = u0; up[1] = u1; up[2] = u2;
  d = make_float2(dd.x, dd.y);
#else
  m[0] = *(const float4*)c0; m[1] = *(const float4*)c1; m[2] = *(const float4*)c2;
  up[0] = c0[upOff]; up[1] = c1[upOff]; up[2] = c2[upOff];
  d = *(const float2*)dp;
#endif
}

__host__ __device__ __forceinline__ void pair_write_entries(float* t, float d0, int code0, float d1, int code1) {
#if defined(__HIP_DEVICE_COMPILE__)
  const float f0 = bits_float(code0), f1 = bits_float(code1);
  v4f e = {d0, f0, d1, f1};
  asm volatile("ds_write_b128 %0, %1" ::"v"(lds_addr(t)), "v"(e) : "memory");
#else
  t[0] = d0; t[1] = bits_float(code0); t[2] = d1; t[3] = bits_float(code1);
#endif
}

// three consecutive entries of two columns of the table
__host__ __device__ __forceinline__ void pair_read_b(float (&dv)[2][3], int (&cd)[2][3], const float* e0, const float* e1) {
#if defined(__HIP_DEVICE_COMPILE__)
  v4f a0, a1;
  pair_v2f b0, b1;
  asm volatile(
      "ds_read_b128 %0, %4\n\t"
      "ds_read_b64 %1, %4 offset:16\n\t"
      "ds_read_b128 %2, %5\n\t"
      "ds_read_b64 %3, %5 offset:16\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(a0), "=&v"(b0), "=&v"(a1), "=&v"(b1)
      : "v"(lds_addr(e0)), "v"(lds_addr(e1))
      : "memory");
  // (element by element through scalars: a bit cast applied directly to a vector element takes element 0)
  const float f[2][6] = {{a0.x, a0.y, a0.z, a0.w, b0.x, b0.y}, {a1.x, a1.y, a1.z, a1.w, b1.x, b1.y}};
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      dv[w][q] = f[w][2 * q];
      cd[w][q] = float_bits(f[w][2 * q + 1]);
    }
#else
  const float* e[2] = {e0, e1};
  for (int w = 0; w < 2; ++w)
    for (int q = 0; q < 3; ++q) {
      dv[w][q] = e[w][2 * q];
      cd[w][q] = float_bits(e[w][2 * q + 1]);
    }
#endif
}

// Stage A for thread (wr, s): output column a + wr, output rows 2s and 2s + 1.  xs: the tile's x columns, dys: its dzdy,
// tab: the table being written (entries of two floats: dzdy, then the winner's code 4 * column + row as an integer;
// -1: routes nothing).
__host__ __device__ __forceinline__ void pair_stage_a(const PairP& p, const PairTile& g, int wr, int s, const float* xs,
                                                      const float* dys, float* tab) {
  const int ow = g.a + wr;
  const bool colLive = ow < p.outW;
  const bool colCopy = g.shift && wr == 0;  // window column 0 is padding, read as a copy of column 1
  const bool rowCopy = s == 0;              // window row 0 of output row 0 is padding, read as a copy of row 1
  const int base = 2 * wr * p.H + 4 * s;
  int o[3];
  o[0] = colCopy ? base : base - g.shift * p.H;
  o[1] = base + p.H - g.shift * p.H;
  o[2] = base + 2 * p.H - g.shift * p.H;
  float v[3][5];  // rows 4s - 1 ... 4s + 3 of the window's three columns
  float4 m[3];
  float up[3];
  float2 d;
  pair_read_a(m, up, d, xs + o[0], xs + o[1], xs + o[2], rowCopy ? 0 : -1, dys + wr * p.outH + 2 * s);
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    v[j][0] = up[j];
    v[j][1] = m[j].x;
    v[j][2] = m[j].y;
    v[j][3] = m[j].z;
    v[j][4] = m[j].w;
  }
  int code[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    float best = -INFINITY;
    int cd = -1;
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const float e = v[j][2 * q + i];
        cd = e > best ? (4 * j + i) : cd;
        best = pair_max(best, e);
      }
    code[q] = cd;
  }
  // a copy that won stands for its original
  code[0] = (rowCopy && code[0] >= 0 && (code[0] & 3) == 0) ? code[0] + 1 : code[0];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    code[q] = (colCopy && code[q] >= 0 && code[q] < 4) ? code[q] + 4 : code[q];
    code[q] = (colLive && 2 * s + q < p.outH) ? code[q] : -1;
  }
  pair_write_entries(tab + 2 * (wr * p.tpitch + 2 * s), d.x, code[0], d.y, code[1]);
}

// Stage B for one 16-byte cell: dzdx rows 4s ... 4s+3 of the tile's column cr (column 2a + cr of the plane).  An even
// column is window column 1 of output column wr = cr / 2 only; an odd one is window column 2 of output column wr and
// then window column 0 of output column wr + 1.  Output rows 2s + q, q ascending, within each.
__host__ __device__ __forceinline__ void pair_stage_b(const PairP& p, int cr, int s, const float* tab, float (&c)[4]) {
  const int wr = cr >> 1;
  const bool odd = cr & 1;
  float dv[2][3];
  int cd[2][3];
  pair_read_b(dv, cd, tab + 2 * (wr * p.tpitch + 2 * s), tab + 2 * ((wr + 1) * p.tpitch + 2 * s));
  const int base0 = odd ? 8 : 4, base1 = odd ? 0 : 64;  // (64: no code has that value, the second column takes no part)
#pragma unroll
  for (int r = 0; r < 4; ++r) c[r] = 0.f;
  // row r of the cell is row i = r + 1 - 2q of window q
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int q = 0; q < 3; ++q)
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const int r = 2 * q + i - 1;
        if (r >= 0 && r <= 3) {
          const float t = c[r] + dv[w][q];
          c[r] = cd[w][q] == (w == 0 ? base0 : base1) + i ? t : c[r];
        }
      }
}

typedef __attribute__((address_space(3))) void* pair_lds_ptr;

// Tile order.  Workgroups that start together do not finish together: the hardware serves the oldest wavefronts of a
// compute unit first, and with equal shares the first of a unit's four workgroups is done after 31 us, the last after
// 41 (timestamps per workgroup), so a bandwidth-bound kernel runs its last fifth on a fraction of its workgroups.  The
// workgroups of a compute unit therefore get unequal shares of the unit's tiles, in proportion to the speeds measured
// (PairP::share).  Workgroups b, b + Q, b + 2Q, ... (Q = grid / workgroups per unit) are the ones the dispatcher puts
// on one compute unit, in that order, when the whole grid is resident (read back from the hardware id registers); the
// result does not depend on that, only the balance does.  (Handing the tiles out at run time instead -- an atomic add
// per tile on a counter per XCD, per compute unit or per workgroup with stealing, drawn ahead by a wavefront of its own
// -- was 1.5 to 5 times slower: an atomic that returns a value takes 2-5 us here beside the streams of loads.)
template <int NL, int STAGES>
__global__ __launch_bounds__(256) void pool_max_backward_pairs(float* __restrict__ dx, const float* __restrict__ x,
                                                                const float* __restrict__ dy, PairP p) {
  extern __shared__ float smem[];
  // layout: stages of (xChunks + dyChunks) KB | 2 tables
  const int stageFloats = (p.xChunks + p.dyChunks) * (kChunk / 4);
  constexpr int D = STAGES - 1;  // tiles in flight behind the one being worked on
  float* const tables = smem + STAGES * stageFloats;
  const int tableFloats = 2 * (p.L + 2) * p.tpitch;  // one table: an entry is two floats; L + 1 window columns and one
                                                      // more that even cells read and never use
  const int tid = (int)threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

  // ---- this workgroup's XCD and its tiles: planes are dealt round-robin to the XCDs (hardware deals workgroup b to XCD
  //      b mod 8), so the tiles of a plane, which read each other's border columns, meet behind one L2, and the chip as a
  //      whole works on one contiguous stretch of memory
  const int G = (int)gridDim.x / p.nx, xcd = (int)blockIdx.x % p.nx;
  const int planesHere = (p.planes - xcd + p.nx - 1) / p.nx;
  const int tilesHere = planesHere * p.tilesPerPlane;
  // the group that shares a compute unit, and with it a pool of tiles: g0 + m S, m = 0, 1, ... in memory order.  Member
  // `self` takes the pool positions m whose residue 39 m mod 64 lies in [shareLo, shareHi): share / 64 of them, evenly
  // spread (39 is coprime to 64: every run of 64 positions has each residue once).
  const int Q = (int)gridDim.x / p.perCu, gid = (int)blockIdx.x % Q, self = (int)blockIdx.x / Q;
  const int S = G / p.perCu, g0 = gid / p.nx;
  const int shareLo = p.share[self], shareHi = p.share[self + 1];
  int scan = 0;  // pool positions looked at so far
  auto next_tile = [&]() -> int {  // this workgroup's next tile; >= tilesHere: none left (and none ever after)
    for (;;) {
      const int m = scan;
      const int t = g0 + S * m;
      if (t >= tilesHere) return 0x7fffffff;
      ++scan;
      const int r = (39 * m) & 63;
      if (r >= shareLo && r < shareHi) return t;
    }
  };

  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)p.xBytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t dr = __builtin_amdgcn_make_buffer_rsrc((void*)dy, 0, (int)p.dyBytes, 0x00020000);

  // Loads of tile t into stage `st`: chunk slots wave, wave + 4, ... (x first, then dzdy).  Nothing is issued for a tile
  // that does not exist or for slots past the stage's chunks: the waits below count real loads only.
  const int chunks = p.xChunks + p.dyChunks;
  const int waveLoads = (chunks - wave + 3) / 4;
  auto issue = [&](int t, int st) {
    if (t >= tilesHere) return;
    const PairTile g = pair_tile(p, xcd, t);
    float* stage = smem + st * stageFloats;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int c = 4 * i + wave;  // chunk slot: uniform per wavefront
      if (c < p.xChunks) {
        const unsigned vo = g.xOff + (unsigned)(c * kChunk + lane * 16);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (pair_lds_ptr)(stage + c * (kChunk / 4)), 16, (int)vo, 0, 0, 0);
      } else if (c < chunks) {
        const unsigned vo = g.dyOff + (unsigned)((c - p.xChunks) * kChunk + lane * 16);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(dr, (pair_lds_ptr)(stage + c * (kChunk / 4)), 16, (int)vo, 0, 0, 0);
      }
    }
  };

  // tables: every code -1 (the two entries past a column's last output row stay that way)
  for (int i = tid; i < 2 * tableFloats; i += 256) tables[i] = bits_float(-1);

  // tile numbers of this workgroup's tiles k ... k+1+D in t[0 ... 1+D] (a number >= tilesHere: no such tile, nor any
  // after it)
  int t[D + 2];
  t[0] = 0;
#pragma unroll
  for (int i = 0; i <= D; ++i) t[i + 1] = next_tile();
#pragma unroll
  for (int i = 0; i < D; ++i) issue(t[i + 1], i);
  int wr, s;
  p.byH4.divmod(tid, &wr, &s);
  const bool inA = wr <= p.L;
  int cr1, s1;  // this thread's second cell of a tile
  p.byH4.divmod(tid + 256, &cr1, &s1);

  // Stores count with the loads (one counter, decremented in issue order), so the wait must know how many memory
  // instructions this wavefront issued after the loads it waits for: the next tile's loads (if there is a next tile)
  // and the 0, 1 or 2 stores of the iteration before.
  const bool oddW = p.W > 2 * p.outW;  // one column behind the last window (plan: at most one)
  int stores = 0;
  for (int k = -1;; ++k) {
    // here: t[0] = tile k (k >= 0), t[1] = tile k+1, ... t[1+D] = tile k+1+D
    {
      // tile k+1 has landed: this wavefront's share first, then (barrier) everybody's
      int after = stores;
#pragma unroll
      for (int i = 2; i <= D; ++i) after += t[i] < tilesHere ? waveLoads : 0;
      switch (after) {
        case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    issue(t[1 + D], (k + 1 + D) % STAGES);
    if (t[1] < tilesHere && inA) {
      const PairTile g = pair_tile(p, xcd, t[1]);
      const float* stage = smem + ((k + 1) % STAGES) * stageFloats;
      pair_stage_a(p, g, wr, s, stage, stage + p.xChunks * (kChunk / 4), tables + ((k + 1) & 1) * tableFloats);
    }
    stores = 0;
    if (k >= 0) {
      const PairTile g = pair_tile(p, xcd, t[0]);
      // the tile's cells in memory order: cell m is rows 4 (m mod H/4) ... of the tile's column m / (H/4); a wavefront's
      // store is 1 KB of consecutive memory.  (The column behind the last window of a plane of odd width takes part as
      // one more even column: the window column it looks up does not exist and never wins.)
      const int cells = (2 * g.nPairs + ((oddW && g.a + g.nPairs == p.outW) ? 1 : 0)) * p.H4;
      float* out = dx + g.outOff;
      const float* tab = tables + (k & 1) * tableFloats;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const bool mine = tid + 256 * u < cells;
        stores += __builtin_amdgcn_ballot_w64(mine) != 0 ? 1 : 0;
        if (mine) {
          float c[4];
          pair_stage_b(p, u == 0 ? wr : cr1, u == 0 ? s : s1, tab, c);
          stream_store4((float4*)out + tid + 256 * u, make_float4(c[0], c[1], c[2], c[3]));
        }
      }
    }
    if (t[1] >= tilesHere) break;  // tile k was this workgroup's last
#pragma unroll
    for (int i = 0; i <= D; ++i) t[i] = t[i + 1];
    t[1 + D] = next_tile();
  }
}

// Shares of a compute unit's tiles, in 64ths, for its workgroups in the order they were started.  Measured with equal
// shares on the 112x112x64x32 case, four workgroups per unit: they finished after 30.7, 34.5, 37.6 and 41.2 us.
static void pair_shares(PairP* p, bool weighted) {
  static const int four[4] = {18, 17, 15, 14};
  if (p->perCu < 1 || p->perCu > 8) p->perCu = 1;
  int sum = 0;
  for (int j = 0; j < 9; ++j) p->share[j] = 64;
  p->share[0] = 0;
  for (int j = 0; j < p->perCu; ++j) {
    sum += (weighted && p->perCu == 4) ? four[j] : (64 * (j + 1)) / p->perCu - (64 * j) / p->perCu;
    p->share[j + 1] = sum;
  }
}

// Shape of a launch.  False when the problem does not fit the kernel.
static bool pair_plan(const mcn_pool_geom* g, int outH, int outW, int cus, int blocksPerCu, int cols, int stages, bool weighted, PairP* out,
                      unsigned* grid, size_t* lds, int* loads) {
  if (g->poolH != 3 || g->poolW != 3 || g->strideY != 2 || g->strideX != 2 || g->padTop != 1 || g->padLeft != 1) return false;
  if (g->H % 4 != 0 || g->H < 4 || g->W < 2 || outH < 1 || outW < 1) return false;
  // no window reaches past the last row or column (no copies are made there); dzdy columns start 16-byte aligned
  if (2 * (outH - 1) + 1 > g->H - 1 || 2 * (outW - 1) + 1 > g->W - 1 || outH != g->H / 2 || outH % 4 != 0) return false;
  if (g->W - 2 * outW > 1) return false;  // (at most one column behind the last window)
  const long long planes = (long long)g->C * g->N;
  const unsigned long long xBytes = (unsigned long long)planes * g->H * g->W * 4, dyBytes = (unsigned long long)planes * outH * outW * 4;
  if (planes < 1 || planes >= (1ll << 31) || xBytes >= 0xC0000000ull) return false;
  PairP p;
  p.H = g->H; p.W = g->W; p.outH = outH; p.outW = outW; p.H4 = g->H / 4;
  p.planes = (int)planes;
  p.nx = planes >= kNumXcd ? kNumXcd : 1;
  p.tpitch = outH + 2;
  p.stages = stages = stages == 3 ? 3 : 2;
  p.xBytes = (unsigned)xBytes;
  p.dyBytes = (unsigned)dyBytes;
  // Pairs per tile: (L + 1) H/4 threads take part (the window column after the tile's last pair is found again here).
  // Among the few largest L the one with the least bytes through the busiest compute unit: rounds of tiles per
  // workgroup x workgroups per compute unit x bytes of a tile.
  if (cus <= 0) cus = 256;
  const int Lmax = std::min(256 / p.H4 - 1, outW);
  if (Lmax < 1) return false;
  const long long planesPerXcd = (planes + p.nx - 1) / p.nx;
  long long bestCost = -1, bestPerXcd = 0;
  size_t bestBytes = 0;
  for (int L = Lmax; L >= std::max(1, Lmax - 3); --L) {
    if (cols > 0 && L != std::min(cols, Lmax)) continue;
    const int tiles = (outW + L - 1) / L;
    const int xc = ((2 * L + 3) * p.H * 4 + kChunk - 1) / kChunk, dc = ((L + 1) * outH * 4 + kChunk - 1) / kChunk;
    if ((xc + dc + 3) / 4 > 4) continue;
    const size_t bytes = (size_t)stages * (xc + dc) * kChunk + (size_t)2 * (L + 2) * p.tpitch * 8;
    if (bytes > 150 * 1024) continue;
    const int fit = (int)std::min<size_t>(std::max<size_t>((160 * 1024) / (bytes + 512), 1), 8);
    const int perCu = blocksPerCu > 0 ? std::min(blocksPerCu, fit) : fit;
    const long long perXcd = std::max<long long>(1, std::min<long long>(planesPerXcd * tiles, (long long)cus * perCu / p.nx));
    const long long rounds = (planesPerXcd * tiles + perXcd - 1) / perXcd;
    const long long cost = rounds * perCu * ((long long)(4 * L + 3) * p.H + (long long)(L + 1) * outH);
    if (bestCost < 0 || cost < bestCost) {
      bestCost = cost;
      bestPerXcd = perXcd;
      bestBytes = bytes;
      p.L = L;
      p.tilesPerPlane = tiles;
      p.xChunks = xc;
      p.dyChunks = dc;
      // (groups of workgroups that share a compute unit exist when the grid is exactly what the chip holds at once)
      p.perCu = (perXcd * p.nx == (long long)cus * perCu && cus % p.nx == 0) ? perCu : 1;
    }
  }
  if (bestCost < 0) return false;
  const int nl = (p.xChunks + p.dyChunks + 3) / 4;
  pair_shares(&p, weighted);
  p.byH4 = FastDiv(p.H4);
  p.byTiles = FastDiv(p.tilesPerPlane);
  const size_t bytes = bestBytes;
  const long long perXcd = bestPerXcd;
  if (perXcd * p.nx >= (1ll << 31) || planesPerXcd * p.tilesPerPlane >= (1ll << 31)) return false;
  *grid = (unsigned)(perXcd * p.nx);
  *lds = bytes;
  *loads = nl;
  *out = p;
  return true;
}

}  // namespace

// Launches the kernel when the problem fits it.  Returns true when the work was enqueued.
bool pool_max_backward_pairs_launch(hipStream_t s, const mcn_pool_geom* g, int outH, int outW, float* derInput,
                                    const float* x, const float* derOutput, int accumulate) {
  if (accumulate || !aligned16(derInput) || !aligned16(x) || !aligned16(derOutput)) return false;
  if (!tunable("pool_pairs", 0)) return false;  // (measured equal to 2% slower than the streaming kernel: by request only)
  PairP p;
  unsigned blocks = 0;
  size_t lds = 0;
  int nl = 0;
  // (as many workgroups per compute unit as fit, tile width chosen, three stages, weighted shares)
  if (!pair_plan(g, outH, outW, device_compute_units(), 0, 0, 3, true, &p, &blocks, &lds, &nl))
    return false;
  typedef void (*Kernel)(float*, const float*, const float*, PairP);
  static const Kernel kernels[2][4] = {
      {pool_max_backward_pairs<1, 2>, pool_max_backward_pairs<2, 2>, pool_max_backward_pairs<3, 2>, pool_max_backward_pairs<4, 2>},
      {pool_max_backward_pairs<1, 3>, pool_max_backward_pairs<2, 3>, pool_max_backward_pairs<3, 3>, pool_max_backward_pairs<4, 3>}};
  const Kernel kernel = kernels[p.stages - 2][nl - 1];
  static std::atomic<size_t> raised[kMaxDevices][2][4];
  const int dev = current_device();
  if (lds > 64 * 1024 && (dev < 0 || dev >= kMaxDevices || lds > raised[dev][p.stages - 2][nl - 1].load(std::memory_order_acquire))) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    if (dev >= 0 && dev < kMaxDevices) raised[dev][p.stages - 2][nl - 1].store(lds, std::memory_order_release);
  }
  const dim3 grid(blocks), block(256);
  KernelTimer timer("pool_backward_pairs", s);
  hipLaunchKernelGGL(kernel, grid, block, lds, s, derInput, x, derOutput, p);
  return true;
}

}  // namespace mcn
