// Shared host/device helpers of the gfx950 back-end: error reporting, launch checks, index helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/mcn_hip.h"

namespace mcn {

// Records a message for the calling thread and returns `code` (numerically a vl::ErrorCode).
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Looks at the launch status without synchronising (the reference peeks the same way,
// bits/datacu.cu:356-371): a failed launch becomes MCN_DEVICE_ERROR with the HIP text.
int check_launch(const char* what);

int tunable(const char* name, int fallback);

// Ordinal of the current device (-1 on error) and its number of compute units (cached per device; -1 on error).
// Per-device host state (function attributes already raised, addresses of device symbols) is kept in arrays of
// kMaxDevices entries.
constexpr int kMaxDevices = 64;
int current_device();
int device_compute_units();
bool stream_beside(hipStream_t s);  // marked by mcn_stream_beside: its launches take one workgroup slot per CU

// Brackets one kernel launch with HIP events when live profiling of that kernel family is switched on
// (mcn_profile_begin); costs one relaxed load otherwise.  Construct right before the launch, on its stream.
class KernelTimer {
 public:
  KernelTimer(const char* kernel, hipStream_t stream);
  ~KernelTimer();

 private:
  int slot;
  hipStream_t stream;
};

inline hipStream_t as_stream(mcn_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int div_up(long long a, long long b) { return (int)((a + b - 1) / b); }

// Division of a non-negative 31-bit integer by a run-time constant without the ~35-instruction hardware
// sequence: q = (mulhi(n, mul) + n) >> shift with mul = floor(2^32 (2^shift - d) / d) + 1, shift = ceil(log2 d).
// Exact for 0 <= n < 2^31, 1 <= d < 2^31.  Built on the host, passed to kernels by value.
struct FastDiv {
  unsigned mul, shift;
  int d;
  FastDiv() : mul(0), shift(0), d(1) {}
  explicit FastDiv(int divisor) : d(divisor < 1 ? 1 : divisor) {
    shift = 0;
    while ((1ll << shift) < d) ++shift;
    mul = (unsigned)((((1ull << 32) * ((1ull << shift) - (unsigned long long)d)) / (unsigned long long)d) + 1ull);
  }
  __host__ __device__ __forceinline__ int div(int n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    return (int)((__umulhi((unsigned)n, mul) + (unsigned)n) >> shift);
#else
    return (int)(((((unsigned long long)(unsigned)n * mul) >> 32) + (unsigned)n) >> shift);
#endif
  }
  __host__ __device__ __forceinline__ void divmod(int n, int* q, int* r) const {
    *q = div(n);
    *r = n - *q * d;
  }
};

constexpr int kWave = 64;      // CDNA wavefront width
constexpr int kNumXcd = 8;     // MI355X: 8 accelerator dies, each with its own L2

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs.  This maps a hardware block id to a
// logical id such that each XCD walks one contiguous range of logical ids, so neighbouring tiles
// (which share halos / operands) meet in the same L2.
__device__ __forceinline__ int xcd_contiguous_id(int bid, int nblocks) {
  const int q = nblocks / kNumXcd, r = nblocks % kNumXcd;
  const int xcd = bid % kNumXcd, i = bid / kNumXcd;
  return xcd * q + (xcd < r ? xcd : r) + i;
}

// 16-byte accesses for data that is touched once per kernel: the non-temporal hint keeps such streams from
// displacing re-used lines (halos, accumulators being merged) in the L2 of each XCD.
#ifndef MCN_NT_STORE
#define MCN_NT_STORE 1
#endif
#ifndef MCN_NT_LOAD
#define MCN_NT_LOAD 0
#endif
typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void stream_store4(float4* p, const float4 v) {
#if MCN_NT_STORE
  v4f t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, (v4f*)p);
#else
  *p = v;
#endif
}
__device__ __forceinline__ float4 stream_load4(const float4* p) {
#if MCN_NT_LOAD
  const v4f t = __builtin_nontemporal_load((const v4f*)p);
  return make_float4(t.x, t.y, t.z, t.w);
#else
  return *p;
#endif
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

}  // namespace mcn
