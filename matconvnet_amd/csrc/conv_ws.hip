// Weights-stationary implicit-GEMM convolution for small filter banks (forward and backward-data of layers whose
// whole packed bank wt[R][co] fits in LDS: the 1x1 and 3x3 layers of a ResNet bottleneck, for instance).
//
// The tiled kernel of conv_mfma.hip stages both operands through LDS with a barrier per 16 reduction rows; with
// short reductions (R = 64 ... 576) and 64-channel tiles its workgroups spend most of their time waiting for the
// one step of loads they have in flight.  Here
//   * a persistent workgroup copies the bank into LDS once (up to 150 KB; one workgroup per CU), laid out
//     [channel block][R][32 WA] so that every weight-fragment read is "lane base + immediate";
//   * each wavefront then works alone, with no barriers: it takes units of 32 pixels x (32 WA) output channels;
//     the pixel operand of v_mfma_f32_32x32x2_f32 is exactly "lane = pixel (l32), half = reduction row (kh)", so it
//     is loaded from global memory straight into the register the MFMA reads -- 32 consecutive pixels of one
//     channel per half-wave, 128-byte runs;
//   * those loads are buffer loads: the per-lane offset is the pixel (+ tap shift), the scalar offset is the
//     channel, and a lane whose shifted pixel falls outside the image simply uses an offset beyond the tensor,
//     for which the hardware returns 0 -- no masks, no selects, no branches, no out-of-bounds access possible;
//   * four register buffers of 8 reduction pairs rotate, so three groups of loads are in flight behind the one
//     being multiplied, and the stream of loads runs on from one unit of a wavefront into its next without
//     draining (the per-unit address arithmetic is done beside the stores of the unit before);
//   * a finished unit is written by 16 straight-line buffer stores per 32 channels ("lane offset + scalar
//     offset"), invisible to the compiler's wait bookkeeping so that they do not drain the load stream;
//   * the loop carries about one vector-ALU instruction per 8 MFMAs (vector-ALU work is what competes with the
//     matrix pipe for the SIMD: with 5 per MFMA an earlier form of this kernel reached only half the MFMA rate);
//   * units are dealt so that every SIMD of the chip gets the same number of them to within one, and the channel
//     blocks of one pixel block go to neighbouring wavefronts of one workgroup (the pixels come from HBM once).
// Reduction order: chunks of 16 channels, the taps inside a chunk (the packed bank's order), pairs of rows per MFMA, sequential accumulation in fp32 like the
// tiled kernel.
#include "conv_common.hpp"

#include <algorithm>
#include <atomic>

namespace mcn {
namespace {

constexpr int kDepth = 8;       // reduction pairs per group: Cin must be a multiple of 16 so a group stays inside a tap
constexpr int kMaxTapsWs = 128;

struct WsP {
  int nUnits;        // pixel blocks x channel blocks, of one slice
  int slices;        // the bank is cut into this many slices of output channels; a workgroup holds one of them
  int chanBlocks;    // channel blocks of 32 WA channels per slice: coutPad / (32 WA slices)
  int groups;        // R / (2 kDepth)
  int groupsPerTap;  // Cin / (2 kDepth)
  unsigned inBytes;  // size of the gathered tensor
  int deepCopy;
  FastDiv byCB, byRow;  // byRow: 8 WA = 16-byte vectors per bank row of one channel block
};

// STATS (WA = 1, one slice, no bias, beta = 0, every wavefront on one channel block for good): the kernel also sums what
// it stores, and its square, per output channel -- the first pass of a batch normalisation that follows, taken from
// the accumulators instead of re-reading the tensor.  Each lane keeps fp32 running sums of its pixels over the
// wavefront's units (a few values each), the wavefront adds its lanes up once at the end, the wavefronts of a workgroup
// that share a channel block add theirs through LDS in a fixed order, and the workgroup writes one fp64 partial per
// channel (alpha must be 1): p.stats[(channel * p.statGroups + workgroup) * 2 + {0: sum, 1: sum of squares}].  Which
// pixels a workgroup sums is fixed by the launch shape: same bits every run.
// Sum over a row of 16 lanes, left in the row's lane 15: v += v shifted right by 1, 2, 4, 8 lanes inside the row (zeros
// shift in), each a single vector add with a lane-shift modifier.
__device__ __forceinline__ float row_sum16(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true));
  return v;
}

// ADD (no bias, alpha = 1, beta = 0, whole channel blocks only): the epilogue adds a second term from another tensor,
// gated by one bit per element (PixP::addend, store_block_masked_add).
template <int WA, bool TAPS, int THREADS, bool STATS = false, bool ADD = false>
__global__ __launch_bounds__(THREADS) void conv_ws_mfma(float* __restrict__ out, const float* __restrict__ in,
                                                        const float* __restrict__ wt, const float* __restrict__ bias,
                                                        PixP p, WsP w) {
  static_assert(!STATS || WA == 1, "channel sums are kept for one 32-channel block per wavefront");
  static_assert(!(STATS && ADD), "one extra at a time");
  extern __shared__ float smem[];
  float* wtL = smem;  // [chanBlocks][R][32 WA]
  constexpr int ROW = 32 * WA;                     // floats per bank row of one channel block
  float* statsL = smem + (size_t)p.R * p.coutPad;  // STATS: [wavefront][2 rows of lanes][32 channels][2], behind the bank

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // (readfirstlane tells the compiler what it cannot see: a wavefront's index is the same in all its lanes, so
  // everything derived from it -- the unit, the loop bounds, the scalar load offsets -- lives in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kh = lane >> 5;
  const int IHW = p.IH * p.IW;

  // Banks too large for LDS are cut into slices of output channels: workgroup w holds slice w % slices and works
  // through all the pixels for those channels (the pixels are then read once per slice, from L2 after the first).
  const int wgAll = TAPS ? xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x) : (int)blockIdx.x;
  const int slice = w.slices > 1 ? wgAll % w.slices : 0;
  const int wg = w.slices > 1 ? wgAll / w.slices : wgAll;          // this workgroup's place among those of its slice
  const int nWg = (int)gridDim.x / w.slices;
  const int cbBase = slice * w.chanBlocks;                         // first channel block of the slice

  // ---- units of this wavefront.  The channel blocks of one pixel block go to neighbouring wavefronts of one
  // workgroup, which reach them at about the same time.  Pixel blocks are dealt slot-major (slot = wavefront /
  // channel blocks), so that consecutive pixel blocks sit on different CUs and every SIMD of the chip gets the
  // same number of units to within one.
  constexpr int wavesPerGroup = THREADS / 64;
  const int sib = w.chanBlocks <= wavesPerGroup ? w.chanBlocks : 1;  // siblings side by side (else one wave, all blocks in turn)
  const int slots = wavesPerGroup / sib;
  const int unitStep = nWg * slots * sib;
  // (workgroup ids are dealt round-robin to the 8 XCDs; with taps, numbering them XCD by XCD puts neighbouring
  // pixel blocks, whose taps reach into each other's columns, behind the same L2: the 3x3 layer of the block then
  // fetches 30 MB per launch through the fabric instead of 128 MB.  Without taps nothing is shared and spreading
  // neighbours over the XCDs measured 5% faster.)
  int unit = ((wave / sib) * nWg + wg) * sib + (wave % sib);
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, (int)w.inBytes, 0x00020000);
  const int planeBytes = IHW * 4;

  // ---- the loader: a stream of groups (16 reduction rows x 32 pixels) that runs three groups ahead of the MFMAs
  // and passes from one unit of this wavefront to the next without draining.  Its state:
  unsigned voff;     // byte offset of this lane's pixel and reduction half at tap shift 0 (kOutside: idle lane)
  int ihB, iwB;      // gathered coordinates at tap shift 0
  unsigned voffN;    // the same three for the unit after the one being loaded: worked out beside the stores of a
  int ihBN, iwBN;    // finished unit, so that the loop itself carries no address arithmetic
  int tapL = 0, giL = 0;  // tap and 16-channel chunk of the next group (taps innermost: see conv_pack_weights)
  unsigned voTap;    // per-lane offset of that tap's pixels (a register of its own for the whole tap: recomputed
                     // per group, the register allocator handed its register to a load result, and every group
                     // then waited for all loads in flight before it could form the next offset)

  // lane geometry of unit u (the pixels do not depend on the channel block); past the last unit every lane idles
  auto setup_next = [&](int u) {
    const int m = w.byCB.div(u) * 32 + l32;
    const bool mvalid = u < w.nUnits && m < p.M;
    int n, q, ow, oh;
    p.byQ.divmod(mvalid ? m : 0, &n, &q);
    if (!TAPS) {
      // (one tap at shift 0, unit strides, output plane = input plane: the pixel's place in its image is q itself)
      ihBN = iwBN = 0;
      voffN = mvalid ? (unsigned)(n * p.inImg + q + kh * IHW) * 4u : kOutside;
      return;
    }
    p.byOH.divmod(q, &ow, &oh);
    ihBN = mvalid ? oh * p.sy : -0x40000000;  // (an idle lane fails every "row inside the image" test)
    iwBN = ow * p.sx;
    voffN = mvalid ? (unsigned)(n * p.inImg + oh * p.sy + p.IH * iwBN + kh * IHW) * 4u : kOutside;
  };

  // The loader's tap, as scalars kept up to date by additions: row index inside the filter column and the tap's
  // shift (dh, dw) of the gathered position.  (A table in LDS cost a read, two readfirstlanes and the wait for
  // them in every group.)
  int tapRow = 0, dhL = p.dhBase, dwL = p.dwBase;
  // per-lane offset of the pixels at shift (dh, dw): kOutside where the shifted pixel is not in the image
  auto tap_offset = [&](int dh, int dw) -> unsigned {
    if (!TAPS) return voff;
    const bool ok = (unsigned)(ihB + dh) < (unsigned)p.IH && (unsigned)(iwB + dw) < (unsigned)p.IW;
    return ok ? voff + (unsigned)((dh + p.IH * dw) * 4) : kOutside;
  };

  typedef float vbuf __attribute__((ext_vector_type(kDepth)));
  vbuf b0, b1, b2, b3;

  // Loads the stream's next group into DST and advances the loader.  Past this wavefront's last unit the loads
  // still go out, with the "outside" offset (they fetch nothing and return 0): the instruction stream is the same
  // on every path, which lets the compiler count exactly how many younger loads may stay in flight at each MFMA.
#define WS_LOAD_NEXT(DST)                                                                                 \
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
      if (++giL == w.groupsPerTap) {                                                                      \
        giL = 0;                                                                                          \
        voff = voffN;                                                                                     \
        ihB = ihBN;                                                                                       \
        iwB = iwBN;                                                                                       \
        if (!TAPS) voTap = voff;                                                                          \
      }                                                                                                   \
    }                                                                                                     \
    if (TAPS) voTap = tap_offset(dhL, dwL);                                                               \
  } while (0)

  // multiplies the stream's oldest group (operands CUR, group G of the unit in hand) after putting one more
  // group in flight into FREE
#define WS_STEP_C(G, CUR, FREE, ZEROC)                                                                            \
  {                                                                                                               \
    WS_LOAD_NEXT(FREE);                                                                                           \
    const float* aG_ = aG + (G) * (2 * kDepth * ROW);                                                             \
    constexpr int HALF_ = kDepth / 2;                                                                             \
    _Pragma("unroll") for (int h_ = 0; h_ < 2; ++h_) {                                                            \
      float av_[HALF_][WA];                                                                                       \
      _Pragma("unroll") for (int d_ = 0; d_ < HALF_; ++d_)                                                        \
        _Pragma("unroll") for (int a_ = 0; a_ < WA; ++a_) av_[d_][a_] = aG_[(2 * (h_ * HALF_ + d_)) * ROW + a_ * 32]; \
      _Pragma("unroll") for (int d_ = 0; d_ < HALF_; ++d_)                                                        \
        _Pragma("unroll") for (int a_ = 0; a_ < WA; ++a_)                                                         \
          acc[a_] = __builtin_amdgcn_mfma_f32_32x32x2f32(av_[d_][a_], CUR[h_ * HALF_ + d_],                     \
                                                         (ZEROC) && h_ == 0 && d_ == 0 ? zero16 : acc[a_], 0, 0, 0); \
    }                                                                                                             \
    /* Pins the step's MFMAs before the next step's loads.  Left free, the compiler lifts those loads over the */ \
    /* last MFMA, which still reads a register of the buffer they fill; the load then gets a fresh register    */ \
    /* and the loop copies it back at its end, after waiting for every load in flight.                         */ \
    _Pragma("unroll") for (int a_ = 0; a_ < WA; ++a_) asm volatile("" : "+v"(acc[a_])::"memory");                 \
  }
#define WS_STEP(G, CUR, FREE) WS_STEP_C(G, CUR, FREE, false)

  // The stream's first three groups go out before the bank is copied: they land while the copy runs, instead of the
  // whole chip asking for its first pixels at once after it (the loads return in order, so the copy's own waits cover
  // them; block step 0.711 -> 0.700 ms.  Only the first group ahead of the copy and the other two behind it, so that
  // the bank does not queue behind 24 loads: 0.708 -> 0.702).  Wavefronts without units issue nothing and leave after
  // the barrier.
  const bool mine = wave < slots * sib && unit < w.nUnits;
  if (mine) {
    setup_next(unit);
    voff = voffN;
    ihB = ihBN;
    iwB = iwBN;
    setup_next(unit + unitStep);
    voTap = tap_offset(dhL, dwL);
    WS_LOAD_NEXT(b0);
    WS_LOAD_NEXT(b1);
    WS_LOAD_NEXT(b2);
  }

  // ---- once per workgroup: the bank, re-laid by channel block
  {
    const int perBlock = p.R * (ROW / 4);  // 16-byte vectors per channel block
    const int n4 = perBlock * w.chanBlocks;
    // (four vectors in flight per thread: one at a time, every round trip to L2 would be paid in full; the empty
    // asm keeps the compiler from sinking each load into the branch that guards its store)
    auto fetch = [&](int i) -> v4f {
      i = min(i, n4 - 1);
      const int cbk = i / perBlock;  // (one-time code: a plain division)
      const int rem = i - cbk * perBlock;
      int r, c4;
      w.byRow.divmod(rem, &r, &c4);
      return *(const v4f*)(wt + (size_t)r * p.coutPad + (cbBase + cbk) * ROW + c4 * 4);
    };
    int i0 = tid;
    // As many vectors in flight per thread as the bank has for it, up to twelve (a 147 KB bank is nine per thread at
    // 1024 threads: one round trip to L2 instead of three, 80.1 -> 78.3 us on 3x3x64x64 over 56x56x64x32); a pass never
    // asks for more than four vectors beyond the bank's end (those re-read its last vector, all threads the same one,
    // which costs more than it looks: a pass of twelve over a bank of eight per thread lost 1-1.5 us)
    for (; w.deepCopy && i0 + 8 * THREADS < n4; i0 += 12 * THREADS) {
      v4f v[12];
#pragma unroll
      for (int k = 0; k < 12; ++k) v[k] = fetch(i0 + k * THREADS);
      asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                   "+v"(v[9]), "+v"(v[10]), "+v"(v[11]));
#pragma unroll
      for (int k = 0; k < 12; ++k)
        if (i0 + k * THREADS < n4) ((v4f*)wtL)[i0 + k * THREADS] = v[k];
    }
    for (; w.deepCopy && i0 + 4 * THREADS < n4; i0 += 8 * THREADS) {
      v4f v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = fetch(i0 + k * THREADS);
      asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (i0 + k * THREADS < n4) ((v4f*)wtL)[i0 + k * THREADS] = v[k];
    }
    for (; i0 < n4; i0 += 4 * THREADS) {
      v4f v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = fetch(i0 + k * THREADS);
      asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (i0 + k * THREADS < n4) ((v4f*)wtL)[i0 + k * THREADS] = v[k];
    }
    if (STATS) statsL[tid] = statsL[tid + THREADS] = 0.f;  // ([THREADS / 64][2 rows][32][2]: wavefronts without units leave zeros)
  }
  __syncthreads();

  if (wave >= slots * sib) return;
  // (STATS: sib = chanBlocks, so a wavefront's channel block is wave % sib for all its units)
  float s1[STATS ? 16 : 1], s2[STATS ? 16 : 1];
  auto write_stats = [&]() {
    if (!STATS) return;
    // the 32 lanes of a half-wave hold the same 16 channels for 32 different pixels.  Rows of 16 lanes are added up
    // inside the vector unit (four shifted adds: lane 15 of a row ends with the row's sum), the two rows of a half meet
    // in LDS.
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s1[r] = row_sum16(s1[r]);
      s2[r] = row_sum16(s2[r]);
    }
    if ((lane & 15) == 15) {
      const int row = l32 >> 4;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 4 * kh + 8 * (r / 4) + r % 4;  // channel inside the block
        statsL[((wave * 2 + row) * 32 + c) * 2] = s1[r];
        statsL[((wave * 2 + row) * 32 + c) * 2 + 1] = s2[r];
      }
    }
    __syncthreads();  // (wavefronts that had no units have left already: the barrier counts the others)
    // wavefront b < sib adds up channel block b: slots in ascending order, lane = channel, in double
    if (wave < sib && lane < 32) {
      double t1 = 0.0, t2 = 0.0;
      for (int j = 0; j < slots; ++j)
        for (int row = 0; row < 2; ++row) {
          t1 += (double)statsL[(((j * sib + wave) * 2 + row) * 32 + lane) * 2];
          t2 += (double)statsL[(((j * sib + wave) * 2 + row) * 32 + lane) * 2 + 1];
        }
      const int c = wave * 32 + lane;
      if (c < p.Cout) {
        double* o = p.stats + ((size_t)c * p.statGroups + wg) * 2;
        o[0] = t1;
        o[1] = t2;
      }
    }
  };
  if (STATS) {
#pragma unroll
    for (int r = 0; r < 16; ++r) s1[r] = s2[r] = 0.f;
  }
  // (STATS: wavefront b < sib writes the workgroup's partial of channel block b, so it stays to the end even without
  // units; the host admits only launches in which every workgroup has units for its first wavefronts)
  if (unit >= w.nUnits) return;

  const bufrsrc orsrc = make_bufrsrc(out, p.outBytes);
  const int plane = p.outPlane * 4;

  floatx16 acc[WA];  // (written whole by a unit's first matrix instructions)
  floatx16 zero16;
#pragma unroll
  for (int r = 0; r < 16; ++r) zero16[r] = 0.f;
  int pb, cb;
  w.byCB.divmod(unit, &pb, &cb);  // unit = pixel block * chanBlocks + channel block
  const float* aLane = wtL + (size_t)cb * p.R * ROW + kh * ROW + l32;
  const float* aG = aLane;  // weight rows of the group in hand

  // One flat loop over this wavefront's whole stream, four groups per turn (the host admits only reductions of
  // a multiple of 4 groups, so a unit ends at the end of a turn with the four buffers back in place).
  const int quadsPerUnit = w.groups >> 2;
  while (true) {
    // a unit's first matrix instruction takes zero as its addend (an operand of the instruction: no sixteen moves per
    // accumulator and unit to clear it); the unit's other turns of four groups follow in a loop of their own
    WS_STEP_C(0, b0, b3, true)
    WS_STEP(1, b1, b0)
    WS_STEP(2, b2, b1)
    WS_STEP(3, b3, b2)
    aG += 4 * (2 * kDepth * ROW);
    for (int quadsLeft = quadsPerUnit - 1; quadsLeft != 0; --quadsLeft) {
      WS_STEP(0, b0, b3)
      WS_STEP(1, b1, b0)
      WS_STEP(2, b2, b1)
      WS_STEP(3, b3, b2)
      aG += 4 * (2 * kDepth * ROW);
    }

    // ---- stores of the finished unit (the next unit's first three groups are already in flight)
    const int mo = pb * 32 + l32;
    const int cbOut = cbBase + cb;  // the channel block's place in the whole bank
    // (STATS and ADD launches have a descriptor-covered output whose channel blocks are whole or padding only, by
    // contract: they always take this branch -- a block of padding stores to the "outside" offset, i.e. nothing, and
    // adds zeros to the sums -- so the test is known at compile time, the other branch is gone, and with it the copies
    // of the thirty-two running sums that the compiler made where the two branches met, every unit)
    const bool whole = (cbOut + 1) * ROW <= p.Cout;
    if ((STATS || ADD) || (p.outBytes != 0 && whole)) {
      // whole channel blocks inside the tensor: straight-line stores through a buffer descriptor
      int n, q;
      p.byQ.divmod(mo < p.M ? mo : 0, &n, &q);
      const unsigned vo =
          mo < p.M && whole ? (unsigned)(n * p.outImg + out_pixel_offset(p, q) + 4 * kh * p.outPlane) * 4u : kOutside;
      if (ADD) {
        const bufrsrc arsrc = make_bufrsrc(p.addend, p.outBytes), brsrc = make_bufrsrc(p.addBits, p.outBytes >> 5);
#pragma unroll
        for (int a = 0; a < WA; ++a) store_block_masked_add(acc[a], orsrc, arsrc, brsrc, vo, (cbOut * ROW + a * 32) * plane, plane);
      } else {
#pragma unroll
        for (int a = 0; a < WA; ++a)
          store_block(acc[a], orsrc, vo, (cbOut * ROW + a * 32) * plane, plane, p.alpha, p.beta,
                      bias ? bias + cbOut * ROW + a * 32 : nullptr, kh);
      }
      if (STATS) {
        // what was stored is the accumulator itself (alpha = 1; lanes past the last pixel hold zeros: their loads
        // fetched nothing)
        // (as instructions that update the sums where they are: the compiler put the results into fresh registers and
        // copied all 32 back at the end of every unit)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          asm("v_add_f32 %0, %0, %1" : "+v"(s1[r]) : "v"(acc[0][r]));
          asm("v_fmac_f32 %0, %1, %1" : "+v"(s2[r]) : "v"(acc[0][r]));
        }
      }
    } else if (mo < p.M) {
      int n, q;
      p.byQ.divmod(mo, &n, &q);
      float* o = out + (size_t)n * p.outImg + out_pixel_offset(p, q);
#pragma unroll
      for (int a = 0; a < WA; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int co = cbOut * ROW + a * 32 + 8 * (r / 4) + 4 * kh + (r % 4);
          if (co < p.Cout) {
            float v = p.alpha * acc[a][r];
            if (p.beta != 0.f) v = fmaf(p.beta, o[(size_t)co * p.outPlane], v);
            if (bias) v += bias[co];
            o[(size_t)co * p.outPlane] = v;
          }
        }
    }
    unit += unitStep;
    if (unit >= w.nUnits) break;
    setup_next(unit + unitStep);  // (the loader is already inside `unit`)
    w.byCB.divmod(unit, &pb, &cb);
    aLane = wtL + (size_t)cb * p.R * ROW + kh * ROW + l32;
    aG = aLane;
  }
  write_stats();
#undef WS_STEP
#undef WS_STEP_C
#undef WS_LOAD_NEXT
}

template <int WA, bool TAPS, int THREADS, bool STATS = false, bool ADD = false>
int launch(hipStream_t s, const char* who, int blocks, size_t lds, float* out, const float* in, const float* wt,
           const float* bias, const PixP& p, const WsP& w) {
  // largest dynamic LDS size this instantiation has been opted into, per device (concurrent callers may both opt in:
  // the attribute call is idempotent, the atomic only keeps the bookkeeping whole)
  static std::atomic<size_t> raised[kMaxDevices];
  const int dev = current_device();
  if (lds > 64 * 1024 && (dev < 0 || dev >= kMaxDevices || lds > raised[dev].load(std::memory_order_acquire))) {
    if (hipFuncSetAttribute((const void*)conv_ws_mfma<WA, TAPS, THREADS, STATS, ADD>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess) {
      (void)hipGetLastError();
      return fail(MCN_DEVICE_ERROR, "%s: cannot reserve %zu bytes of LDS", who, lds);
    }
    if (dev >= 0 && dev < kMaxDevices) {
      size_t seen = raised[dev].load(std::memory_order_relaxed);
      while (seen < lds && !raised[dev].compare_exchange_weak(seen, lds, std::memory_order_release)) {
      }
    }
  }
  KernelTimer timer("conv_ws_mfma", s);
  hipLaunchKernelGGL((conv_ws_mfma<WA, TAPS, THREADS, STATS, ADD>), dim3((unsigned)blocks), dim3(THREADS), lds, s, out, in, wt, bias, p, w);
  return check_launch(who);
}

// One workgroup per CU: sixteen wavefronts (4 per SIMD, 128 registers each) for the narrow units; eight for WA = 4,
// whose 64 accumulator registers plus operands need more than 128.  (Banks of up to 78 KB used to get two workgroups of
// eight wavefronts per CU; one of sixteen copies the bank once per CU instead of twice and measured 1.5-2 us faster per
// launch on the 1x1 layers of a 56x56x256x32 bottleneck, 42-48 us each.)
template <int WA, bool TAPS>
int dispatch(hipStream_t s, const char* who, int cus, size_t lds, float* out, const float* in, const float* wt,
             const float* bias, const PixP& p, const WsP& w) {
  constexpr int THREADS = WA == 4 ? 512 : 1024;
  if (p.addend) return launch<WA, TAPS, THREADS, false, true>(s, who, cus, lds, out, in, wt, bias, p, w);
  if constexpr (WA == 1) {
    if (p.stats) return launch<1, TAPS, 1024, true>(s, who, cus, lds, out, in, wt, bias, p, w);
  }
  return launch<WA, TAPS, THREADS>(s, who, cus, lds, out, in, wt, bias, p, w);
}

}  // namespace

namespace {

// How the weights-stationary kernel would run `p`: unit width, slices, workgroups.  False: it does not take this
// product.  wantStats: only shapes that can also sum their output per channel (see the kernel).
struct WsPlan {
  int WA, cus, statGroups;
  bool taps;
  size_t lds;
  WsP w;
};

bool plan_ws(const PixP& p, bool wantStats, WsPlan* plan) {
  if (tunable("conv_no_ws", 0)) return false;
  if (p.Cin % (2 * kDepth) != 0 || p.R % (8 * kDepth) != 0 || p.T > kMaxTapsWs || p.coutPad % 32 != 0) return false;
  // the bank, or the smallest power-of-two number of slices of it (each a multiple of 32 output channels), in 150 KB
  const int maxSlices = wantStats ? 1 : 8;
  int slices = 1;
  while (slices <= maxSlices && ((size_t)p.R * (p.coutPad / slices) * sizeof(float) > 150 * 1024 || p.coutPad % (32 * slices) != 0)) {
    if (p.coutPad % (32 * slices * 2) != 0) return false;
    slices *= 2;
  }
  if (slices > maxSlices) return false;
  // every slice gathers all the pixels again: with a strided gather (half of each line fetched unused) the tiled
  // kernel, which gathers once, is the faster one
  if (slices > 1 && (p.sy > 1 || p.sx > 1) && !tunable("conv_ws_sliced_strided", 0)) return false;
  const int coutSlice = p.coutPad / slices;
  const size_t lds = (size_t)p.R * coutSlice * sizeof(float);
  // byte offsets into the gathered tensor must stay below the "outside" offset
  const long long inBytes = ((long long)(p.N - 1) * p.inImg + (long long)p.Cin * p.IH * p.IW) * 4;
  if (inBytes >= (long long)kOutside) return false;

  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  if (cus % slices != 0) return false;  // (every slice gets the same number of workgroups)
  const long long simds = (long long)cus * 4;
  const long long pixelBlocks = ((long long)p.M + 31) / 32;

  // channels per wavefront: the widest unit that still spreads evenly over the SIMDs (wider units amortise the
  // pixel loads over more MFMAs; narrower ones balance better)
  const int minUnits = tunable("conv_ws_min_units", 0);
  int WA = wantStats ? 1 : tunable("conv_ws_wa", 0);
  if (WA != 1 && WA != 2 && WA != 4) {
    double best = 0;
    for (int cand : {4, 2, 1}) {
      if (coutSlice % (32 * cand) != 0) continue;
      const long long units = pixelBlocks * (p.coutPad / (32 * cand));
      const double balance = (double)units / (double)(((units + simds - 1) / simds) * simds);
      const double issue = cand == 4 ? 0.96 : (cand == 2 ? 0.94 : 0.90);
      // under four units per SIMD a wide unit no longer pays: the loads of a few long units per SIMD are hidden worse
      // than those of many short ones (stride classes of 3x3 /2 128->128: 130 -> 118 us with the narrowest), so any
      // shape that fills the SIMDs four deep wins over one that does not, and among those that do not the narrowest
      const double score = units >= 4 * simds ? balance * issue : 0.01 / cand;
      if (score > best) {
        best = score;
        WA = cand;
      }
    }
  }
  if (coutSlice % (32 * WA) != 0) return false;
  WsP w;
  w.slices = slices;
  w.chanBlocks = coutSlice / (32 * WA);
  const long long units = pixelBlocks * w.chanBlocks;  // per slice
  // too little work to occupy even half of the SIMDs: leave it to the tiled kernel, which can split its reduction
  if (units >= (1ll << 30) || units * slices < (minUnits > 0 ? (long long)minUnits : simds / 2)) return false;
  w.nUnits = (int)units;
  w.groups = p.R / (2 * kDepth);
  w.groupsPerTap = p.Cin / (2 * kDepth);
  w.inBytes = (unsigned)inBytes;
  w.deepCopy = 1;
  w.byCB = FastDiv(w.chanBlocks);
  w.byRow = FastDiv(8 * WA);
  plan->WA = WA;
  plan->cus = cus;
  plan->taps = !(p.T == 1 && p.dhBase == 0 && p.dwBase == 0 && p.sy == 1 && p.sx == 1 && p.IH == p.OH && p.IW == p.OW);
  plan->lds = lds;
  plan->w = w;
  plan->statGroups = 0;
  if (wantStats) {
    // the sums are taken where whole 32-channel blocks are stored through the output's buffer descriptor: no block
    // may be partial (a block of padding only has nothing to sum) and the output must be under 2 GiB, or some
    // channels' sums would stay zero
    if (p.Cout % 32 != 0 || p.outBytes == 0) return false;
    // every wavefront must stay on one channel block: the channel blocks sit side by side in a workgroup
    const int wavesPerGroup = 16;
    if (wavesPerGroup % w.chanBlocks != 0 || p.beta != 0.f || p.alpha != 1.f) return false;
    const int nWg = cus;
    // the first wavefronts of every workgroup (slot 0) must have a unit: they write the workgroup's partials
    if (units < (long long)nWg * w.chanBlocks) return false;
    if (lds + (size_t)wavesPerGroup * 128 * sizeof(float) > 160 * 1024) return false;
    plan->lds = lds + (size_t)wavesPerGroup * 128 * sizeof(float);
    plan->statGroups = nWg;
  }
  return true;
}

}  // namespace

int conv_ws_stat_groups(const PixP& p) {
  WsPlan plan;
  return plan_ws(p, true, &plan) ? plan.statGroups : 0;
}

int conv_ws_launch(hipStream_t s, const char* who, float* out, const float* in, const float* wt, const float* bias,
                   const PixP& p, int* handled) {
  *handled = 0;
  WsPlan plan;
  const bool wantStats = p.stats != nullptr;
  if (!plan_ws(p, wantStats, &plan) || (wantStats && (bias || plan.statGroups != p.statGroups))) {
    if (wantStats) return fail(MCN_UNSUPPORTED, "%s: this product cannot sum its output per channel", who);
    return MCN_SUCCESS;
  }
  if (p.addend || p.addQuery) {
    // the second term of the epilogue: dense whole 32-channel blocks of a tensor a buffer descriptor covers, planes of
    // whole 32-bit mask words
    const bool fits = !wantStats && !bias && p.alpha == 1.f && p.beta == 0.f && p.dense && p.outBytes != 0 && p.Cout % 32 == 0 &&
                      p.Cout == p.coutPad && p.outPlane % 32 == 0 && p.outImg % 32 == 0 && (p.addQuery || p.addBits);
    if (p.addQuery) {
      *p.addQuery = fits ? 1 : 0;
      *handled = 1;
      return MCN_SUCCESS;
    }
    if (!fits) return fail(MCN_UNSUPPORTED, "%s: this product cannot add a masked second term in its epilogue", who);
  }
  const int WA = plan.WA, cus = plan.cus;
  const size_t lds = plan.lds;
  const WsP& w = plan.w;
  int rc;
  if (plan.taps) rc = WA == 4 ? dispatch<4, true>(s, who, cus, lds, out, in, wt, bias, p, w)
                      : (WA == 2 ? dispatch<2, true>(s, who, cus, lds, out, in, wt, bias, p, w)
                                 : dispatch<1, true>(s, who, cus, lds, out, in, wt, bias, p, w));
  else rc = WA == 4 ? dispatch<4, false>(s, who, cus, lds, out, in, wt, bias, p, w)
            : (WA == 2 ? dispatch<2, false>(s, who, cus, lds, out, in, wt, bias, p, w)
                       : dispatch<1, false>(s, who, cus, lds, out, in, wt, bias, p, w));
  *handled = 1;
  return rc;
}

}  // namespace mcn
