// Geometry shared by the convolution kernels.
#pragma once

#include "mcn_internal.hpp"

#include <vector>

namespace mcn {

struct ConvP {
  int H, W, C, N;
  int FH, FW, FC, K;
  int sy, sx, pt, pl, dy, dx;
  int outH, outW;
  int groups, Kg;  // Kg = filters per group
};

// Validates like the MEX driver (vl_nnconv.cu:269-342) and fills the derived fields.
int conv_setup(const mcn_conv_geom* g, const char* who, ConvP* p);

// direct (one accumulator per output element) kernels: any stride / dilation / padding / groups
int conv_forward_direct(hipStream_t s, const ConvP& p, float* y, float outMult, const float* x, float inMult,
                        const float* f, const float* b);
int conv_backward_data_direct(hipStream_t s, const ConvP& p, float* dx, float dxMult, const float* f, const float* dy);
int conv_backward_filter_direct(hipStream_t s, const ConvP& p, float* df, const float* x, const float* dy);

// The taps of a stored FH x FW filter that take part in one product: (i0 + a*iStep, j0 + b*jStep), a < nI, b < nJ
// (all of them for a plain layer; one stride class for the backward-data product of a strided layer).
struct TapSet {
  int FH, FW;            // the filter as stored
  int i0, iStep, nI;
  int j0, jStep, nJ;
};

// One re-laying of (part of) a filter bank into the order the MFMA kernels read: a launch of conv_pack_weights, or
// one entry of a batched launch.  Plain data: it crosses the C ABI as mcn_conv_pack_job.
struct PackJob {
  float* wt;
  const float* f;
  TapSet taps;
  int Cin, Cout, rPad, coutPad, backward, tapMajor;
  unsigned firstBlock, blocks;  // workgroups [firstBlock, firstBlock + blocks) of a batched launch
};

// Filter banks packed ahead of the calls that use them.  The products of a layer visit their banks in a fixed
// order (groups, then stride classes); every bank takes a 256-byte aligned slot of the caller's buffer in that
// order, so planning, packing and using agree on where each one lies.
struct PackCtx {
  enum Mode { kPlan, kPack, kUse };
  Mode mode;
  char* base;                  // the caller's buffer (null when only the size is wanted)
  size_t capacity, offset;
  std::vector<PackJob>* jobs;  // kPlan: the jobs are appended here instead of being launched
};

// The sum over reduction splits that finishes a filter gradient (conv_wgrad_reduce), as data: one entry of a batched
// launch.  Plain data: it crosses the C ABI as mcn_conv_reduce_job.
struct ReduceJob {
  float* df;
  const float* partials;
  size_t n;               // elements of the bank
  int splits, tapMajor, C, T;
  unsigned firstBlock, blocks;
};

// Filter gradients whose final sum is deferred: the matrix kernel leaves its partial banks in the caller's buffer
// (one 256-byte aligned slot per filter group, in group order) and the sums of many layers run in one launch later.
struct ReduceCtx {
  char* base;
  size_t capacity, offset;
  std::vector<ReduceJob>* jobs;  // not null: the jobs are appended here
  bool launch;                   // false: plan only (sizes and jobs), nothing is launched
};

// MFMA implicit-GEMM kernels (groups == 1).  *_supported says whether the fast path covers `p`.
bool conv_mfma_forward_supported(const ConvP& p);
bool conv_mfma_backward_data_supported(const ConvP& p);
bool conv_mfma_backward_filter_supported(const ConvP& p);
// first layers (few input channels, 32 or 64 filters): filter gradient and, from the same pass, bias gradient
// (conv_first.hip); dB may be null
bool conv_first_backward_filter_supported(const ConvP& p);
size_t conv_first_workspace_bytes(const ConvP& p);
// (their forward product; and their input gradient at stride 1, on vector FMAs: at most four channels come out)
bool conv_first_forward_supported(const ConvP& p);
int conv_first_forward(hipStream_t s, const ConvP& p, float* y, const float* x, const float* f, const float* bias);
bool conv_first_backward_data_supported(const ConvP& p);
int conv_first_backward_data(hipStream_t s, const ConvP& p, float* dx, const float* f, const float* dy);
int conv_first_backward_filter(hipStream_t s, const ConvP& p, float* dF, float* dB, const float* x, const float* dy, void* ws,
                               size_t wsBytes);
size_t conv_mfma_workspace_bytes(const ConvP& p, int product);
// stats / statGroups: also write per-channel partial sums of y and y^2 (see PixP::stats); statQuery: plan only
int conv_forward_mfma(hipStream_t s, const ConvP& p, float* y, float outMult, const float* x, float inMult,
                      const float* f, const float* b, void* ws, size_t wsBytes, PackCtx* pk = nullptr,
                      double* stats = nullptr, int statGroups = 0, int* statQuery = nullptr);
// addend / addBits: a masked second term added in the epilogue (see PixP::addend); addQuery: plan only
int conv_backward_data_mfma(hipStream_t s, const ConvP& p, float* dx, float dxMult, const float* f, const float* dy,
                            void* ws, size_t wsBytes, PackCtx* pk = nullptr, const float* addend = nullptr,
                            const unsigned* addBits = nullptr, int* addQuery = nullptr);
int conv_pack_batch(hipStream_t s, const PackJob* deviceJobs, int nJobs, unsigned totalBlocks);
int conv_backward_filter_mfma(hipStream_t s, const ConvP& p, float* df, const float* x, const float* dy, void* ws,
                              size_t wsBytes, ReduceCtx* deferred = nullptr);
int conv_reduce_batch(hipStream_t s, const ReduceJob* deviceJobs, int nJobs, unsigned totalBlocks);

// Parameters of the pixel-major products (forward / backward-data): out[co, m] = sum_R wt[R][co] * in[ci(R), pixel(m) + tap(R)]
struct PixP {
  int IH, IW, Cin;    // grid and channels of the gathered tensor
  int OH, OW, Cout;   // grid and channels of the produced tensor
  int N;
  int FH, T;          // filter height, taps = FH*FW
  int sy, sx;         // gathered row = oh*sy + dh(tap)
  int dhBase, dhStep, dwBase, dwStep;
  int R;              // reduction length = T*Cin
  int coutPad;        // row pitch of wt
  int M;              // OH*OW*N (< 2^31)
  float alpha, beta;
  FastDiv byQ, byOH, byT;  // Q = OH*OW; T = taps
  int advC, advT;          // 16 = advC*T + advT (reduction rows per step)
  unsigned outBytes;       // bytes from `out` to the end of the produced tensor, or 0 when >= 2 GiB (no buffer descriptor)
  // tiled kernel, loads straight into LDS: bytes of the gathered tensor and of the packed bank (both < 2 GiB), else 0
  unsigned inBytes = 0, wtBytes = 0;
  // Where things lie, in elements.  The gathered tensor: image n, channel ci at in + n*inImg + ci*IH*IW.  The produced
  // tensor: pixel (oh, ow) of image n, channel co at out + n*outImg + co*outPlane + outOff + oh*outSH + ow*outSW.
  // A plain layer has inImg = Cin*IH*IW, outImg = Cout*OH*OW, outPlane = OH*OW, outOff = 0, outSH = 1, outSW = OH
  // (dense = 1: the pixel offset is the pixel index itself); a filter group sees a slice of the channels of a
  // wider tensor, a stride class of a strided layer's backward-data product a sub-grid of the pixels.
  int inImg, outImg, outPlane, outOff, outSH, outSW, dense;
  // Split reduction (tiled kernel only; 1 = none): workgroup `split` multiplies steps [split*stepsPerSplit, ...) of
  // 16 rows and writes its partial result to out + split*partStride (dense layout, alpha = 1, beta = 0, no bias);
  // conv_pix_reduce then adds the partials up.  For layers with few output pixels and a long reduction
  // (fully-connected layers above all), which would otherwise keep a handful of workgroups busy for a long time.
  int rSplits, stepsPerSplit;
  long long partStride;
  // Per-channel sums of the produced tensor taken in the same launch (weights-stationary kernel only): where the
  // partial sums go, and how many of them each channel gets.  statQuery (host only): no launch, just report that
  // number (0: this product has no such form).
  double* stats = nullptr;
  int statGroups = 0;
  int* statQuery = nullptr;
  // A second term added in the epilogue (weights-stationary kernel only, dense whole 32-channel blocks, planes of a
  // multiple of 32 elements, alpha = 1, beta = 0, no bias): out = acc + (bit ? addend : addend*0), addend a tensor of
  // the produced tensor's layout, bit = bit e % 32 of word e / 32 of addBits for element e.  addQuery (host only): no
  // launch, just report whether the product has this form.
  const float* addend = nullptr;
  const unsigned* addBits = nullptr;
  int* addQuery = nullptr;
};

// the pixel's element offset inside its channel plane of the produced tensor
__device__ __forceinline__ int out_pixel_offset(const PixP& p, int q) {
  if (p.dense) return q;
  int ow, oh;
  p.byOH.divmod(q, &ow, &oh);
  return p.outOff + oh * p.outSH + ow * p.outSW;
}

// ------------------------------------------------------------------------------------------------
// Epilogue shared by the pixel-major MFMA kernels
// ------------------------------------------------------------------------------------------------
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int bufrsrc __attribute__((ext_vector_type(4)));

constexpr unsigned kOutside = 0x80000000u;  // buffer offset no tensor handled here reaches (they are < 2 GiB)

// Raw buffer descriptor over `bytes` bytes at `base` (uniform): accesses at offsets >= bytes are dropped (stores)
// or return 0 (loads).
__device__ __forceinline__ bufrsrc make_bufrsrc(const void* base, unsigned bytes) {
  const unsigned long long a = (unsigned long long)base;
  bufrsrc r;
  r.x = (int)(unsigned)(a & 0xffffffffull);
  r.y = (int)(unsigned)((a >> 32) & 0xffffull);
  r.z = (int)bytes;
  r.w = 0x00020000;
  return r;
}

// A store the compiler's memory-wait bookkeeping does not see.  With ordinary stores in flight beside loads it
// can no longer tell which of them the hardware counter is counting and waits for everything at every use of a
// loaded value.  The hardware counter still counts these stores; that only makes the compiler's waits for older
// loads (which return in order among themselves) longer, never shorter.  Store data is read when the
// instruction issues, so the registers can be reused right after.
__device__ __forceinline__ void buffer_store_untracked(float v, unsigned voffset, bufrsrc rsrc, int soffset) {
  asm volatile("buffer_store_dword %0, %1, %2, %3 offen" ::"v"(v), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}

// Writes one wavefront's 32 channels x 32 pixels accumulator block of v_mfma_f32_32x32x2_f32 (register r of lane
// l holds channel 8(r/4) + 4(l/32) + r%4 of pixel l%32):  out = alpha*acc (+ beta*out) (+ bias).
//   rsrc     descriptor of the whole output tensor
//   voffset  byte offset of this lane's pixel in channel 4(l/32) of the block's image (kOutside: lane writes nothing)
//   sblock   byte offset of the block's first channel plane (uniform)
//   plane    bytes per channel plane (uniform)
//   biasBlk  bias of the block's first channel, or null (uniform)
// Straight-line: 16 stores at "lane offset + scalar offset", no per-store address arithmetic in vector registers,
// no per-store branches.
template <bool BETA, bool BIAS>
__device__ __forceinline__ void store_block_as(floatx16 acc, bufrsrc rsrc, unsigned voffset, int sblock, int plane,
                                               float alpha, float beta, const float* biasBlk, int kh) {
  float old[16], bv[16];
  if (BETA) {
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(((unsigned long long)(unsigned)rsrc.x) | ((unsigned long long)(unsigned)rsrc.y << 32)), 0, rsrc.z, rsrc.w);
#pragma unroll
    for (int r = 0; r < 16; ++r)
      old[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rr, (int)voffset, sblock + (8 * (r / 4) + r % 4) * plane, 0));
  }
  if (BIAS) {
#pragma unroll
    for (int r = 0; r < 16; ++r) bv[r] = biasBlk[8 * (r / 4) + 4 * kh + r % 4];
  }
  if (!BETA && !BIAS && alpha == 1.f) {
    // the plain product: the accumulators as they are (1 * x = x: sixteen multiplies less per block, which short
    // reductions -- 32 MFMAs per block with 64 input channels -- notice)
#pragma unroll
    for (int r = 0; r < 16; ++r) buffer_store_untracked(acc[r], voffset, rsrc, sblock + (8 * (r / 4) + r % 4) * plane);
    return;
  }
  // (alpha made opaque here: left visible, the compiler forms the sixteen products before it tests alpha == 1 and the
  // plain product above pays for them as well)
  asm volatile("" : "+s"(alpha));
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float v = alpha * acc[r];
    if (BETA) v = fmaf(beta, old[r], v);
    if (BIAS) v += bv[r];
    buffer_store_untracked(v, voffset, rsrc, sblock + (8 * (r / 4) + r % 4) * plane);
  }
}

__device__ __forceinline__ void store_block(floatx16 acc, bufrsrc rsrc, unsigned voffset, int sblock, int plane,
                                            float alpha, float beta, const float* biasBlk, int kh) {
  if (beta != 0.f) {
    if (biasBlk) store_block_as<true, true>(acc, rsrc, voffset, sblock, plane, alpha, beta, biasBlk, kh);
    else store_block_as<true, false>(acc, rsrc, voffset, sblock, plane, alpha, beta, biasBlk, kh);
  } else if (biasBlk) {
    store_block_as<false, true>(acc, rsrc, voffset, sblock, plane, alpha, beta, biasBlk, kh);
  } else {
    store_block_as<false, false>(acc, rsrc, voffset, sblock, plane, alpha, beta, biasBlk, kh);
  }
}

// out = acc + (bit ? addend : addend*0): the block of store_block with a second term from a tensor of the same layout,
// gated by one bit per element (see PixP::addend).  arsrc / brsrc: descriptors of the addend and of the bit words;
// voffset and sblock as in store_block (plane bytes a multiple of 128, so a lane's bit position is the same for all 16
// channels and the word offset splits into a lane part and a scalar part).
__device__ __forceinline__ void store_block_masked_add(floatx16 acc, bufrsrc rsrc, bufrsrc arsrc, bufrsrc brsrc, unsigned voffset,
                                                       int sblock, int plane) {
  const __amdgpu_buffer_rsrc_t ar = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(((unsigned long long)(unsigned)arsrc.x) | ((unsigned long long)(unsigned)arsrc.y << 32)), 0, arsrc.z, arsrc.w);
  const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(((unsigned long long)(unsigned)brsrc.x) | ((unsigned long long)(unsigned)brsrc.y << 32)), 0, brsrc.z, brsrc.w);
  const unsigned vword = voffset == kOutside ? kOutside : (voffset >> 7) << 2;  // byte offset of the lane's word at scalar offset 0
  const unsigned bit = (voffset >> 2) & 31u;
  float add[16];
  unsigned wd[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int so = sblock + (8 * (r / 4) + r % 4) * plane;
    add[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ar, (int)voffset, so, 0));
    wd[r] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(br, (int)vword, so >> 5, 0);
  }
  // acc + addend * (0 or 1): the product is exact (the addend itself, or the zero, or the NaN, that addend * 0 is), so one
  // fused multiply-add gives the bits of "bit ? addend : addend * 0" added to acc -- three vector instructions per
  // element (bit field, conversion, multiply-add) instead of six
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float gate = (float)__builtin_amdgcn_ubfe(wd[r], bit, 1u);
    buffer_store_untracked(__builtin_fmaf(add[r], gate, acc[r]), voffset, rsrc, sblock + (8 * (r / 4) + r % 4) * plane);
  }
}

// Weights-stationary variant (conv_ws.hip) for filter banks that fit in LDS: wt is the packed bank in the
// 16-channel-chunk order of conv_pack_weights.  Sets *handled when it took the work.
int conv_ws_launch(hipStream_t s, const char* who, float* out, const float* in, const float* wt, const float* bias,
                   const PixP& p, int* handled);
// partial sums per channel it would write when asked to sum its output (PixP::stats); 0: it would not take `p` that way
int conv_ws_stat_groups(const PixP& p);

// Streamed-bank variant (conv_sb.hip) for banks too large for LDS, same packed order.  conv_sb_splits: the reduction
// splits it would use for a product of these extents (0: it does not take them; depends on nothing else, so that the
// workspace can be sized ahead); conv_sb_plan: the same, with the layout conditions checked.  conv_sb_launch: `p` laid
// out as for the tiled kernel (with splits > 1: the partial tensors' dense layout, alpha = 1, beta = 0, no bias).
// conv_sb_tail_bytes: scratch memory an unsplit launch of these extents wants for the tiles of its last, partly
// filled round (0: none); conv_sb_launch takes it as tailWs (nullptr: every tile by one workgroup).
int conv_sb_splits(int Cout, long long M, int R);
size_t conv_sb_tail_bytes(int Cout, long long M, int R);
bool conv_sb_plan(const PixP& p, int* splits);
int conv_sb_launch(hipStream_t s, float* out, const float* in, const float* wt, const float* bias, PixP p, int splits,
                   float* tailWs);

// Products with at most four output channels (conv_few.hip): wt is the packed bank (tapMajor: its row order, see
// conv_pack_weights).  Sets *handled when it took the work.
int conv_few_launch(hipStream_t s, const char* who, float* out, const float* in, const float* wt, const float* bias,
                    const PixP& p, bool tapMajor, int* handled);

}  // namespace mcn
