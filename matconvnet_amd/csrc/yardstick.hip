// Streaming yardstick: plain read-only, write-only and copy kernels of known size over a sweep of launch shapes
// (workgroups, accesses in flight per lane, access width, walk, store hint).  What the best of them reaches with
// cold caches is the measured ceiling the bandwidth-bound operators are reported against beside the nominal
// 8 TB/s, and the copy of known size is what the HBM byte counters of the other kernels are scaled by.
#include "mcn_internal.hpp"

#include <algorithm>

namespace mcn {
namespace {

typedef float v2f __attribute__((ext_vector_type(2)));

template <typename V>
__device__ __forceinline__ float lanes_sum(V v);
template <>
__device__ __forceinline__ float lanes_sum<float>(float v) { return v; }
template <>
__device__ __forceinline__ float lanes_sum<v2f>(v2f v) { return v.x + v.y; }
template <>
__device__ __forceinline__ float lanes_sum<v4f>(v4f v) { return (v.x + v.y) + (v.z + v.w); }

// MODE 0: read src (a value that cannot occur is stored when the sum says so: the loads must happen)
// MODE 1: write dst;  MODE 2: dst = src.
// n: elements of type V.  Every step a workgroup handles UNROLL slabs of 256 elements, all loads first.
// CHUNKED false: the workgroups share the array slab by slab (at any time they cover one contiguous stretch);
// true: each walks a contiguous run of its own.
template <int MODE, typename V, int UNROLL, bool NT, bool CHUNKED>
__global__ __launch_bounds__(256) void yardstick_kernel(V* __restrict__ dst, const V* __restrict__ src, size_t n,
                                                        float* __restrict__ sink) {
  const size_t span = (size_t)256 * UNROLL;
  const size_t steps = (n + span - 1) / span;
  size_t s0, s1, stride;
  if (CHUNKED) {
    s0 = steps * blockIdx.x / gridDim.x;
    s1 = steps * (blockIdx.x + 1) / gridDim.x;
    stride = 1;
  } else {
    s0 = blockIdx.x;
    s1 = steps;
    stride = gridDim.x;
  }
  float total = 0.f;
  V fill;
  for (int k = 0; k < (int)(sizeof(V) / sizeof(float)); ++k) ((float*)&fill)[k] = 1.f;
  for (size_t s = s0; s < s1; s += stride) {
    const size_t base = s * span + threadIdx.x;
    V v[UNROLL];
    if (MODE != 1) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const size_t i = base + (size_t)256 * u;
        v[u] = i < n ? src[i] : fill;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t i = base + (size_t)256 * u;
      if (MODE == 0) total += lanes_sum<V>(v[u]);
      if (MODE == 1 && i < n) {
        if (NT) __builtin_nontemporal_store(fill, dst + i);
        else dst[i] = fill;
      }
      if (MODE == 2 && i < n) {
        if (NT) __builtin_nontemporal_store(v[u], dst + i);
        else dst[i] = v[u];
      }
    }
  }
  if (MODE == 0 && total == -12345.678f) *sink = total;
}

template <int MODE, typename V, int UNROLL>
void launch_nt(hipStream_t s, int blocks, bool nt, bool chunked, V* dst, const V* src, size_t n, float* sink) {
  const dim3 grid((unsigned)blocks), block(256);
  if (nt && chunked) hipLaunchKernelGGL((yardstick_kernel<MODE, V, UNROLL, true, true>), grid, block, 0, s, dst, src, n, sink);
  else if (nt) hipLaunchKernelGGL((yardstick_kernel<MODE, V, UNROLL, true, false>), grid, block, 0, s, dst, src, n, sink);
  else if (chunked) hipLaunchKernelGGL((yardstick_kernel<MODE, V, UNROLL, false, true>), grid, block, 0, s, dst, src, n, sink);
  else hipLaunchKernelGGL((yardstick_kernel<MODE, V, UNROLL, false, false>), grid, block, 0, s, dst, src, n, sink);
}

template <int MODE, typename V>
int launch_unroll(hipStream_t s, int blocks, int unroll, bool nt, bool chunked, V* dst, const V* src, size_t n, float* sink) {
  switch (unroll) {
    case 1: launch_nt<MODE, V, 1>(s, blocks, nt, chunked, dst, src, n, sink); break;
    case 2: launch_nt<MODE, V, 2>(s, blocks, nt, chunked, dst, src, n, sink); break;
    case 4: launch_nt<MODE, V, 4>(s, blocks, nt, chunked, dst, src, n, sink); break;
    case 8: launch_nt<MODE, V, 8>(s, blocks, nt, chunked, dst, src, n, sink); break;
    default: return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: accesses in flight per lane must be 1, 2, 4 or 8");
  }
  return MCN_SUCCESS;
}

template <typename V>
int launch_mode(hipStream_t s, int mode, int blocks, int unroll, bool nt, bool chunked, void* dst, const void* src,
                size_t bytes, float* sink) {
  const size_t n = bytes / sizeof(V);
  switch (mode) {
    case MCN_YARDSTICK_READ: return launch_unroll<0, V>(s, blocks, unroll, nt, chunked, (V*)dst, (const V*)src, n, sink);
    case MCN_YARDSTICK_WRITE: return launch_unroll<1, V>(s, blocks, unroll, nt, chunked, (V*)dst, (const V*)src, n, sink);
    case MCN_YARDSTICK_COPY: return launch_unroll<2, V>(s, blocks, unroll, nt, chunked, (V*)dst, (const V*)src, n, sink);
    default: return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: unknown mode %d", mode);
  }
}

// Matrix-pipe yardstick: every SIMD of the chip gets four wavefronts, each a dependent chain of matrix instructions on
// its own accumulator (what a convolution's inner loop is once its operands are in registers), and nothing else.
// What it reaches is the ceiling the matrix-bound kernels are reported against beside the nominal peak: the chip does
// not hold its nominal clock under such a stream.
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef double doublex4 __attribute__((ext_vector_type(4)));

template <bool F64>
__global__ __launch_bounds__(1024) void mfma_yardstick_kernel(float* __restrict__ sink, int iters) {
  const float a = (float)(threadIdx.x & 63) * 0.001f, b = 1.0f;
  float total = 0.f;
  if (F64) {
    doublex4 acc = {0.0, 0.0, 0.0, 0.0};
    for (int i = 0; i < iters; ++i)
#pragma unroll
      for (int u = 0; u < 16; ++u) acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)a, (double)b, acc, 0, 0, 0);
    total = (float)((acc[0] + acc[1]) + (acc[2] + acc[3]));
  } else {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    for (int i = 0; i < iters; ++i)
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; ++r) total += acc[r];
  }
  if (total == -12345.678f) *sink = total;  // (cannot happen: the chains must be computed all the same)
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" int mcn_mfma_yardstick(mcn_stream_t stream, void* sink, int iters, int isDouble, double* flop) {
  if (!sink || iters < 1 || iters > (1 << 20)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_mfma_yardstick: null sink or iteration count out of range");
  int cus = device_compute_units();
  if (cus <= 0) cus = 256;
  hipStream_t s = as_stream(stream);
  KernelTimer timer("mfma_yardstick_kernel", s);
  if (isDouble) hipLaunchKernelGGL(mfma_yardstick_kernel<true>, dim3((unsigned)cus), dim3(1024), 0, s, (float*)sink, iters);
  else hipLaunchKernelGGL(mfma_yardstick_kernel<false>, dim3((unsigned)cus), dim3(1024), 0, s, (float*)sink, iters);
  // wavefronts x instructions x FLOP per instruction (32x32x2: 4096; 16x16x4: 2048)
  if (flop) *flop = (double)cus * 16.0 * (double)iters * (isDouble ? 16.0 * 2048.0 : 8.0 * 4096.0);
  return check_launch("mcn_mfma_yardstick");
}

extern "C" int mcn_hbm_yardstick(mcn_stream_t stream, void* dst, const void* src, size_t bytes, int mode, int width,
                                 int inFlight, int blocks, int flags) {
  if (bytes == 0) return MCN_SUCCESS;
  if (bytes % 16 != 0) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: size must be a multiple of 16 bytes");
  if (mode != MCN_YARDSTICK_WRITE && !src) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: null source");
  if (!dst) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: null destination (read mode: one float)");
  if ((mode != MCN_YARDSTICK_READ && !aligned16(dst)) || (src && !aligned16(src)))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: buffers must be 16-byte aligned");
  const size_t slabs = (bytes / (size_t)width + 255) / 256;
  if (blocks <= 0) blocks = (int)std::min<size_t>((slabs + (size_t)inFlight - 1) / (size_t)std::max(inFlight, 1), 1u << 30);
  const bool nt = (flags & MCN_YARDSTICK_NONTEMPORAL) != 0, chunked = (flags & MCN_YARDSTICK_CHUNKED) != 0;
  hipStream_t s = as_stream(stream);
  float* sink = (float*)dst;  // read mode: never written in practice
  int rc;
  KernelTimer timer("yardstick_kernel", s);
  switch (width) {
    case 4: rc = launch_mode<float>(s, mode, blocks, inFlight, nt, chunked, dst, src, bytes, sink); break;
    case 8: rc = launch_mode<v2f>(s, mode, blocks, inFlight, nt, chunked, dst, src, bytes, sink); break;
    case 16: rc = launch_mode<v4f>(s, mode, blocks, inFlight, nt, chunked, dst, src, bytes, sink); break;
    default: return fail(MCN_ILLEGAL_ARGUMENT, "mcn_hbm_yardstick: access width must be 4, 8 or 16 bytes");
  }
  if (rc) return rc;
  return check_launch("mcn_hbm_yardstick");
}
