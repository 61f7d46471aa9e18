// Streamed-bank implicit-GEMM convolution (forward and backward-data of layers whose packed bank wt[R][co] is too
// large to sit in LDS: 3x3x256x256 and the deeper layers of a ResNet).
//
// The tiled kernel of conv_mfma.hip stages BOTH operands of every step through LDS: global load, LDS write, barrier,
// LDS read, with the address arithmetic of all four in the loop -- about two vector-ALU instructions per MFMA, and
// vector-ALU work is what competes with the matrix pipe for the SIMD.  Here only the weights go through LDS:
//   * a workgroup of four wavefronts owns 32 WA output channels x 128 pixels; each wavefront multiplies its own 32
//     pixels against all 32 WA channels (WA accumulator blocks of 32 x 32);
//   * the pixel operand of v_mfma_f32_32x32x2_f32 is "lane = pixel, half-wave = reduction row", exactly what one
//     buffer load per lane delivers, so the pixels go from global memory straight into the register the MFMA reads,
//     through four rotating buffers of 8 reduction pairs (three groups of loads in flight behind the one being
//     multiplied), as in the weights-stationary kernel (conv_ws.hip): per-lane offset = pixel (+ tap shift), scalar
//     offset = channel, out-of-image lanes use an offset beyond the tensor and get 0 from the hardware;
//   * the bank streams through a double buffer in LDS, 32 reduction rows x 32 WA channels at a time: every thread
//     fetches WA 16-byte vectors of the next slab (buffer loads: per-thread constant offset + scalar row offset) before
//     the slab in hand is multiplied and parks them in LDS behind it; one LDS-only barrier per slab, which does not
//     wait for the pixel loads in flight; every weight-fragment read is "lane base + immediate";
//   * the loop carries no address arithmetic in vector registers beyond the tap shift (one select per 16 rows).
// Reduction order: the packed bank's (chunks of 16 channels, the taps inside a chunk), pairs of rows per MFMA,
// sequential accumulation in fp32: the same sums in the same order as the tiled and the weights-stationary kernels.
// A long reduction over few pixels is split like the tiled kernel's (partial tensors + conv_pix_reduce).
// A launch whose tiles do not fill the chip's last round (3136 tiles on 768 resident workgroups: four rounds, then 64
// workgroups alone on the chip for as long as a tile takes a wavefront that has its SIMD to itself) hands those last
// tiles to a second launch that splits THEIR reduction over the whole chip (TAIL instantiation: partial tiles into the
// workspace) and a small kernel that adds the partial tiles up in a fixed order (conv_sb_tail_reduce).
#include "conv_common.hpp"

#include <algorithm>

namespace mcn {
namespace {

constexpr int kDepth = 8;   // reduction pairs per group of pixel loads (16 rows: one tap of one 16-channel chunk)

struct SbP {
  int tilesA;         // channel tiles of 32 WA
  int mTiles;         // pixel tiles of 128
  int slabs;          // slabs of this launch's whole reduction: R / 32
  int slabsPerSplit;  // slabs per reduction split (even)
  int groupsPerTap;   // Cin / 16
  unsigned inBytes;   // size of the gathered tensor
  unsigned wtBytes;   // size of the packed bank
  int tileBase;       // TAIL: first tile of the tail (tiles are numbered pixel tile x tilesA + channel tile)
  int tailTiles;      // TAIL: tiles of the tail; workgroup = (split, tile of the tail), split-major
};

// LDS-only barrier: waits for this wave's LDS traffic, not for the global loads in flight
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// kSlab: reduction rows per slab of the bank in LDS (32 or 64: two or four groups); OCC: wavefronts per SIMD the
// register budget is cut for.  TAIL: the launch covers tiles [tileBase, tileBase + tailTiles), each by several
// workgroups that take a slice of the reduction each and leave their 32 WA x 128 sums, as they are, in a tile of
// their own at out[(split * tailTiles + tile) * 32 WA * 128] (channel-major, 128 pixels per channel).
template <int WA, bool TAPS, int kSlab, int OCC, bool TAIL = false>
__global__ __launch_bounds__(256, OCC) void conv_sb_mfma(float* __restrict__ out, const float* __restrict__ in,
                                                    const float* __restrict__ wt, const float* __restrict__ bias,
                                                    PixP p, SbP w) {
  constexpr int CT = 32 * WA;  // channels per workgroup = floats per slab row
  __shared__ float As[2][kSlab * CT];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kh = lane >> 5;
  const int IHW = p.IH * p.IW;

  // tile of this workgroup: the channel tiles of one pixel tile are neighbours (numbered XCD by XCD: they and the
  // neighbouring pixel tiles, whose taps reach into each other's columns, read the same pixels behind one L2)
  int logical = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
  int split = 0;
  if (TAIL) {
    split = logical / w.tailTiles;
    logical -= split * w.tailTiles;
    out += ((size_t)split * w.tailTiles + logical) * (size_t)(CT * 128);
    logical += w.tileBase;
  } else if (p.rSplits > 1) {  // (split-major: the workgroups of one split are neighbours)
    const int tiles = (int)gridDim.x / p.rSplits;
    split = logical / tiles;
    logical -= split * tiles;
    out += (size_t)split * p.partStride;
  }
  const int mt = logical / w.tilesA;
  const int ca = logical - mt * w.tilesA;
  const int slabBegin = split * w.slabsPerSplit;
  const int slabEnd = min(w.slabs, slabBegin + w.slabsPerSplit);
  if (slabBegin >= slabEnd) return;  // (uniform)

  // ---- the pixel loader (see conv_ws.hip): a stream of groups (16 reduction rows x 32 pixels) three groups ahead
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, (int)w.inBytes, 0x00020000);
  const int planeBytes = IHW * 4;
  const int m = mt * 128 + wave * 32 + l32;
  const bool mvalid = m < p.M;
  unsigned voff;  // byte offset of this lane's pixel and reduction half at tap shift 0 (kOutside: idle lane)
  int ihB, iwB;   // gathered coordinates at tap shift 0
  {
    int n, q, ow, oh;
    p.byQ.divmod(mvalid ? m : 0, &n, &q);
    p.byOH.divmod(q, &ow, &oh);
    ihB = mvalid ? oh * p.sy : -0x40000000;  // (an idle lane fails every "row inside the image" test)
    iwB = ow * p.sx;
    voff = mvalid ? (unsigned)(n * p.inImg + oh * p.sy + p.IH * iwB + kh * IHW) * 4u : kOutside;
  }
  // first group of this split: chunk giL of 16 channels, tap tapL
  const int g0 = slabBegin * (kSlab / (2 * kDepth));
  int giL = g0 / p.T, tapL = g0 - giL * p.T;
  int tapRow = tapL % p.FH;
  int dhL = p.dhBase + tapRow * p.dhStep, dwL = p.dwBase + (tapL / p.FH) * p.dwStep;
  int groupsLeft = (slabEnd - slabBegin) * (kSlab / (2 * kDepth));  // past the last one the loads fetch nothing
  auto tap_offset = [&](int dh, int dw) -> unsigned {
    if (!TAPS) return voff;
    const bool ok = (unsigned)(ihB + dh) < (unsigned)p.IH && (unsigned)(iwB + dw) < (unsigned)p.IW;
    return ok ? voff + (unsigned)((dh + p.IH * dw) * 4) : kOutside;
  };
  unsigned voTap = tap_offset(dhL, dwL);

  typedef float vbuf __attribute__((ext_vector_type(kDepth)));
  vbuf b0, b1, b2, b3;

  // Loads the stream's next group into DST and advances the loader.  Past the split's last group the loads still go
  // out, with the "outside" offset: the instruction stream is the same on every path, which lets the compiler count
  // exactly how many younger loads may stay in flight at each MFMA.
#define SB_LOAD_NEXT(DST)                                                                                 \
  do {                                                                                                    \
    const int sbase_ = giL * (2 * kDepth) * planeBytes;                                                   \
    _Pragma("unroll") for (int d_ = 0; d_ < kDepth; ++d_) DST[d_] = __builtin_bit_cast(                   \
        float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voTap, sbase_ + 2 * d_ * planeBytes, 0));  \
    if (TAPS) {                                                                                           \
      dhL += p.dhStep;                                                                                    \
      if (++tapRow == p.FH) {                                                                             \
        tapRow = 0;                                                                                       \
        dhL = p.dhBase;                                                                                   \
        dwL += p.dwStep;                                                                                  \
      }                                                                                                   \
    }                                                                                                     \
    if (++tapL == p.T) {                                                                                  \
      tapL = 0;                                                                                           \
      dwL = p.dwBase;                                                                                     \
      ++giL;                                                                                              \
    }                                                                                                     \
    if (--groupsLeft == 0) {                                                                              \
      voff = kOutside;                                                                                    \
      ihB = -0x40000000;                                                                                  \
    }                                                                                                     \
    voTap = tap_offset(dhL, dwL);                                                                         \
  } while (0)

  // ---- the bank: slab s = rows [32 s, 32 s + 32) x this tile's channels, WA 16-byte vectors per thread
  const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)wt, 0, (int)w.wtBytes, 0x00020000);
  constexpr int ROWS_PER_PASS = 256 / (CT / 4);  // slab rows covered by one vector per thread
  const unsigned voffA = (unsigned)(((tid / (CT / 4)) * p.coutPad + ca * CT + (tid % (CT / 4)) * 4) * 4);
  const int rowBytes = p.coutPad * 4;
  typedef float v4 __attribute__((ext_vector_type(4)));
  constexpr int PASSES = kSlab * (CT / 4) / 256;  // 16-byte vectors of a slab per thread
  v4 pa[PASSES];
  int slabNext = slabBegin;  // the slab the next fetch brings
#define SB_FETCH_SLAB()                                                                                          \
  do {                                                                                                           \
    const unsigned vo_ = slabNext < slabEnd ? voffA : kOutside;                                                  \
    const int sb_ = slabNext * kSlab * rowBytes;                                                                 \
    _Pragma("unroll") for (int j_ = 0; j_ < PASSES; ++j_) pa[j_] = __builtin_bit_cast(                           \
        v4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)vo_, sb_ + j_ * ROWS_PER_PASS * rowBytes, 0));     \
    ++slabNext;                                                                                                  \
  } while (0)
#define SB_STASH_SLAB(BUF)                                                                   \
  do {                                                                                       \
    _Pragma("unroll") for (int j_ = 0; j_ < PASSES; ++j_) *(v4*)&As[BUF][(tid + 256 * j_) * 4] = pa[j_]; \
  } while (0)

  floatx16 acc[WA];
#pragma unroll
  for (int a = 0; a < WA; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  // multiplies the stream's oldest group (operands CUR; group G of the slab in LDS buffer BUF) after putting one more
  // group in flight into FREE
#define SB_STEP(BUF, G, CUR, FREE)                                                                                \
  {                                                                                                               \
    SB_LOAD_NEXT(FREE);                                                                                           \
    const float* aG_ = &As[BUF][(G) * (2 * kDepth * CT) + kh * CT + l32];                                         \
    constexpr int HALF_ = kDepth / 2;                                                                             \
    _Pragma("unroll") for (int h_ = 0; h_ < 2; ++h_) {                                                            \
      float av_[HALF_][WA];                                                                                       \
      _Pragma("unroll") for (int d_ = 0; d_ < HALF_; ++d_)                                                        \
        _Pragma("unroll") for (int a_ = 0; a_ < WA; ++a_) av_[d_][a_] = aG_[(2 * (h_ * HALF_ + d_)) * CT + a_ * 32]; \
      _Pragma("unroll") for (int d_ = 0; d_ < HALF_; ++d_)                                                        \
        _Pragma("unroll") for (int a_ = 0; a_ < WA; ++a_)                                                         \
          acc[a_] = __builtin_amdgcn_mfma_f32_32x32x2f32(av_[d_][a_], CUR[h_ * HALF_ + d_], acc[a_], 0, 0, 0);    \
    }                                                                                                             \
    /* pins the step's MFMAs before the next step's loads: left free, the scheduler lifts those loads over the  */ \
    /* last MFMA, which still reads a register of the buffer they fill                                          */ \
    __builtin_amdgcn_sched_barrier(0);                                                                            \
  }

  // ---- prologue: the first slab into LDS, three groups of pixels in flight
  SB_FETCH_SLAB();
  SB_LOAD_NEXT(b0);
  SB_LOAD_NEXT(b1);
  SB_LOAD_NEXT(b2);
  SB_STASH_SLAB(0);
  lds_barrier();

  // Two slabs per turn (the host admits only splits of an even number of slabs: the four pixel buffers and the two
  // LDS buffers are back in place at the end of a turn).
  for (int turn = (slabEnd - slabBegin) >> 1; turn > 0; --turn) {
    SB_FETCH_SLAB();
    if (kSlab == 32) {
      SB_STEP(0, 0, b0, b3)
      SB_STEP(0, 1, b1, b0)
    } else {
      SB_STEP(0, 0, b0, b3)
      SB_STEP(0, 1, b1, b0)
      SB_STEP(0, 2, b2, b1)
      SB_STEP(0, 3, b3, b2)
    }
    SB_STASH_SLAB(1);
    lds_barrier();
    SB_FETCH_SLAB();
    if (kSlab == 32) {
      SB_STEP(1, 0, b2, b1)
      SB_STEP(1, 1, b3, b2)
    } else {
      SB_STEP(1, 0, b0, b3)
      SB_STEP(1, 1, b1, b0)
      SB_STEP(1, 2, b2, b1)
      SB_STEP(1, 3, b3, b2)
    }
    SB_STASH_SLAB(0);
    lds_barrier();
  }
#undef SB_STEP
#undef SB_STASH_SLAB
#undef SB_FETCH_SLAB
#undef SB_LOAD_NEXT

  // ---- epilogue: lane = pixel, register = channel
  const int coW = ca * CT;
  if (TAIL) {  // (idle lanes and padding channels hold zeros: every load of theirs was outside its tensor)
    const bufrsrc orsrc = make_bufrsrc(out, (unsigned)(CT * 128 * 4));
    const unsigned vo = (unsigned)(wave * 32 + l32 + 4 * kh * 128) * 4u;
#pragma unroll
    for (int a = 0; a < WA; ++a) store_block(acc[a], orsrc, vo, a * 32 * 512, 512, 1.f, 0.f, nullptr, kh);
    return;
  }
  if (p.outBytes != 0 && coW + CT <= p.Cout) {
    const bufrsrc orsrc = make_bufrsrc(out, p.outBytes);
    const int plane = p.outPlane * 4;
    int n, q;
    p.byQ.divmod(mvalid ? m : 0, &n, &q);
    const unsigned vo = mvalid ? (unsigned)(n * p.outImg + out_pixel_offset(p, q) + 4 * kh * p.outPlane) * 4u : kOutside;
#pragma unroll
    for (int a = 0; a < WA; ++a)
      store_block(acc[a], orsrc, vo, (coW + a * 32) * plane, plane, p.alpha, p.beta, bias ? bias + coW + a * 32 : nullptr, kh);
    return;
  }
  if (!mvalid) return;
  int n, q;
  p.byQ.divmod(m, &n, &q);
  float* o = out + (size_t)n * p.outImg + out_pixel_offset(p, q);
#pragma unroll
  for (int a = 0; a < WA; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = coW + a * 32 + 8 * (r / 4) + 4 * kh + (r % 4);
      if (co < p.Cout) {
        float v = p.alpha * acc[a][r];
        if (p.beta != 0.f) v = fmaf(p.beta, o[(size_t)co * p.outPlane], v);
        if (bias) v += bias[co];
        o[(size_t)co * p.outPlane] = v;
      }
    }
}

// out[tile of the tail] = alpha * (sum over the splits, in their order) (+ beta * out) (+ bias): one thread per
// (tile, channel, pixel), pixels fastest
__global__ __launch_bounds__(256) void conv_sb_tail_reduce(float* __restrict__ out, const float* __restrict__ partials,
                                                           const float* __restrict__ bias, PixP p, int tileBase,
                                                           int tailTiles, int splits, int tilesA, int CT) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const int pxl = (int)(idx & 127);
  const long long rest = idx >> 7;
  const int c = (int)(rest % CT);
  const int tl = (int)(rest / CT);
  if (tl >= tailTiles) return;
  const int tile = tileBase + tl;
  const int mt = tile / tilesA, ca = tile - mt * tilesA;
  const long long m = (long long)mt * 128 + pxl;
  const int co = ca * CT + c;
  if (m >= p.M || co >= p.Cout) return;
  const size_t tileFloats = (size_t)CT * 128;
  const float* src = partials + (size_t)tl * tileFloats + (size_t)c * 128 + pxl;
  float sum = 0.f;
  for (int k = 0; k < splits; ++k) sum += src[(size_t)k * tailTiles * tileFloats];
  int n, q;
  p.byQ.divmod((int)m, &n, &q);
  float* o = out + (size_t)n * p.outImg + out_pixel_offset(p, q) + (size_t)co * p.outPlane;
  float v = p.alpha * sum;
  if (p.beta != 0.f) v = fmaf(p.beta, *o, v);
  if (bias) v += bias[co];
  *o = v;
}

template <int WA, int kSlab, int OCC>
void launch(hipStream_t s, bool taps, unsigned blocks, float* out, const float* in, const float* wt, const float* bias,
            const PixP& p, const SbP& w) {
  if (w.tailTiles > 0) {
    KernelTimer timer("conv_sb_mfma_tail", s);
    if (taps) hipLaunchKernelGGL((conv_sb_mfma<WA, true, kSlab, OCC, true>), dim3(blocks), dim3(256), 0, s, out, in, wt, bias, p, w);
    else hipLaunchKernelGGL((conv_sb_mfma<WA, false, kSlab, OCC, true>), dim3(blocks), dim3(256), 0, s, out, in, wt, bias, p, w);
    return;
  }
  KernelTimer timer("conv_sb_mfma", s);
  if (taps) hipLaunchKernelGGL((conv_sb_mfma<WA, true, kSlab, OCC>), dim3(blocks), dim3(256), 0, s, out, in, wt, bias, p, w);
  else hipLaunchKernelGGL((conv_sb_mfma<WA, false, kSlab, OCC>), dim3(blocks), dim3(256), 0, s, out, in, wt, bias, p, w);
}

}  // namespace

// rows per slab of the bank in LDS for a reduction of R rows (a turn of the kernel's loop is two slabs)
static int slab_rows(int R) {
  (void)R;
  return 32;  // (64-row slabs, possible when R is a multiple of 128, measured no faster)
}

int conv_sb_splits(int Cout, long long M, int R) {
  if (R % 64 != 0 || Cout <= 32) return 0;
  const int BA = Cout > 64 ? 128 : 64;
  const int coutPad = (Cout + BA - 1) / BA * BA;
  if ((long long)R * coutPad * 4 >= (long long)kOutside) return 0;
  const long long tiles = ((M + 127) / 128) * (coutPad / BA);
  if (tiles >= (1ll << 30)) return 0;
  // A long reduction over few tiles is split so that the launch fills the chip: two workgroups per compute unit, at
  // least six pairs of slabs each.  Measured against the tiled kernel's own split reduction, forward, 32 images:
  // 3x3x256x256 on 14x14: 99 -> 92 us, 3x3x512x512 on 7x7: 104 -> 93 us; with 64 images (196 tiles and more) the tiled
  // kernel is the faster one (155 against 160 us), so products with more than half a tile per compute unit are left
  // to it.  Inside the whole network (cold caches, the partial tensors' extra traffic) the split form loses: a ResNet-50
  // training step at 32 images went 12.73 -> 12.90 ms, so it is off unless asked for (conv_sb_split).
  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  const int pairs = R / (2 * slab_rows(R));  // pairs of slabs: the unit a split is made of
  const long long want = (long long)cus * 2;
  int s = 1;
  if (tiles < want) {
    const int minPairs = 6;
    s = (int)std::min<long long>((want + tiles - 1) / tiles, std::max(1, pairs / minPairs));
    const int per = (pairs + s - 1) / s;
    s = (pairs + per - 1) / per;
  }
  if (s > 1 && (!tunable("conv_sb_split", 0) || 2 * tiles > cus)) return 0;
  return s;
}

bool conv_sb_plan(const PixP& p, int* splits) {
  *splits = conv_sb_splits(p.Cout, p.M, p.R);
  if (*splits <= 0) return false;
  if (p.Cin % (2 * kDepth) != 0 || p.T > 128 || p.coutPad % 64 != 0 || (p.Cout > 64 && p.coutPad % 128 != 0)) return false;
  const long long inBytes = ((long long)(p.N - 1) * p.inImg + (long long)p.Cin * p.IH * p.IW) * 4;
  return inBytes < (long long)kOutside;
}

namespace {
// The tail of a launch without reduction splits: the tiles left over after the last full round of resident
// workgroups, and the reduction splits their own launch uses.  Depends on the extents only (workspace sizing).
struct SbTail { int tiles, splits; size_t bytes; };
SbTail sb_tail(int Cout, long long M, int R) {
  SbTail t = {0, 0, 0};
  if (!tunable("conv_sb_tail", 1)) return t;
  const int CT = Cout > 64 ? 128 : 64;
  const int coutPad = (Cout + CT - 1) / CT * CT;
  const long long tilesAll = ((M + 127) / 128) * (coutPad / CT);
  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  const int slab = slab_rows(R);
  // resident workgroups per compute unit of the instantiation conv_sb_launch picks (registers: 160 with 128 channels)
  const int asked = tunable("conv_sb_tail_slots", 0);
  const int perCu = asked > 0 ? asked : CT == 128 ? 3 : slab == 64 ? 3 : 4;
  const long long slots = (long long)cus * perCu;
  if (tilesAll <= slots) return t;  // one round or less
  const long long rem = tilesAll % slots;
  if (rem == 0 || 2 * rem > slots) return t;  // a last round at least half full stays as it is
  const int pairs = R / (2 * slab);
  int s = (int)std::min<long long>(slots / rem, pairs / 2);
  s = std::min(s, 16);
  if (s < 2) return t;
  const int per = (pairs + s - 1) / s;
  s = (pairs + per - 1) / per;
  if (s < 2) return t;
  t.tiles = (int)rem;
  t.splits = s;
  t.bytes = (size_t)s * (size_t)rem * CT * 128 * sizeof(float);
  return t;
}
}  // namespace

size_t conv_sb_tail_bytes(int Cout, long long M, int R) {
  return conv_sb_splits(Cout, M, R) == 1 ? sb_tail(Cout, M, R).bytes : 0;
}

int conv_sb_launch(hipStream_t s, float* out, const float* in, const float* wt, const float* bias, PixP p, int splits,
                   float* tailWs) {
  const int CT = p.coutPad % 128 == 0 && p.Cout > 64 ? 128 : 64;
  const int slab = slab_rows(p.R);
  SbP w;
  w.tilesA = p.coutPad / CT;
  w.mTiles = (int)(((long long)p.M + 127) / 128);
  w.slabs = p.R / slab;
  const int pairs = w.slabs / 2;
  w.slabsPerSplit = 2 * ((pairs + splits - 1) / splits);
  w.groupsPerTap = p.Cin / (2 * kDepth);
  w.inBytes = (unsigned)(((long long)(p.N - 1) * p.inImg + (long long)p.Cin * p.IH * p.IW) * 4);
  w.wtBytes = (unsigned)((long long)p.R * p.coutPad * 4);
  w.tileBase = 0;
  w.tailTiles = 0;
  p.rSplits = splits;
  const bool taps = !(p.T == 1 && p.dhBase == 0 && p.dwBase == 0 && p.sy == 1 && p.sx == 1 && p.IH == p.OH && p.IW == p.OW);
  const int occ = 2;  // (wavefronts per SIMD the 128-channel kernel's registers are cut for; 3 measured slower)
  auto dispatch = [&](unsigned blocks, float* o, const float* b, const SbP& ww) {
    if (CT == 128) {
      if (slab == 64) launch<4, 64, 2>(s, taps, blocks, o, in, wt, b, p, ww);
      else if (occ >= 3) launch<4, 32, 3>(s, taps, blocks, o, in, wt, b, p, ww);
      else launch<4, 32, 2>(s, taps, blocks, o, in, wt, b, p, ww);
    } else {
      if (slab == 64) launch<2, 64, 3>(s, taps, blocks, o, in, wt, b, p, ww);
      else launch<2, 32, 4>(s, taps, blocks, o, in, wt, b, p, ww);
    }
  };
  const long long tilesAll = (long long)w.mTiles * w.tilesA;
  const SbTail tail = splits == 1 && tailWs ? sb_tail(p.Cout, p.M, p.R) : SbTail{0, 0, 0};
  if (tail.tiles > 0 && CT == (p.Cout > 64 ? 128 : 64)) {
    // full rounds as they are, then the left-over tiles with their reduction split over the whole chip
    dispatch((unsigned)(tilesAll - tail.tiles), out, bias, w);
    SbP wb = w;
    wb.tileBase = (int)(tilesAll - tail.tiles);
    wb.tailTiles = tail.tiles;
    wb.slabsPerSplit = 2 * ((pairs + tail.splits - 1) / tail.splits);
    dispatch((unsigned)((long long)tail.tiles * tail.splits), tailWs, nullptr, wb);
    KernelTimer timer("conv_sb_tail_reduce", s);
    const long long threads = (long long)tail.tiles * CT * 128;
    hipLaunchKernelGGL(conv_sb_tail_reduce, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, out, tailWs, bias, p,
                       wb.tileBase, tail.tiles, tail.splits, w.tilesA, CT);
    return MCN_SUCCESS;
  }
  dispatch((unsigned)(tilesAll * splits), out, bias, w);
  return MCN_SUCCESS;
}

}  // namespace mcn
