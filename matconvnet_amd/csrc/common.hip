// Error state, tunables and device queries of the gfx950 back-end.
#include "mcn_internal.hpp"

#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace mcn {

namespace {
thread_local char g_message[512] = "";

// Values are read on every launch (several per launch) from any thread and written only by experiments: relaxed
// atomics, no lock; the table itself never changes.
struct Tunable {
  const char* name;
  std::atomic<int> value;
  Tunable(const char* n, int v) : name(n), value(v) {}
};
// Defaults are the values chosen from on-device sweeps; see the per-kernel comments where each is read.
Tunable g_tunables[] = {
    {"conv_sb_split", 0},              // 0: the streamed-bank kernel leaves products whose reduction it would split to the tiled kernel
                                       // (on their own, warm, the split products win 8-11% at 32 images; inside ResNet-50 the step loses 0.17 ms)
    {"conv_sb_tail", 1},               // streamed-bank kernel: the tiles of a partly filled last round get a launch of their own that splits their reduction
    {"conv_sb_tail_slots", 0},         // resident workgroups per compute unit that plan assumes (0: the instantiation's own)
    {"pool_lds_bytes", 16 * 1024},     // LDS tile budget of the pooling-backward kernels
    {"pool_pairs", 0},                 // 1: max pooling backward over 3x3 windows at stride 2, padding 1 by the kernel with direct-to-LDS
                                       // loads and one winner table (pool_pairs.hip) instead of the streaming kernel (equal to 2% slower)
    {"pool_force_gather", 0},          // 1: skip the ordered-pass kernel, use the general tiled gather
    {"bnorm_one_launch_elems", 8192},  // channels of at most this many elements (and >= 128 of them): sums and apply in one launch
    {"conv_no_ws", 0},                 // 1: never use the weights-stationary kernel
    {"conv_first_max_wg", 0},          // > 0: at most this many workgroups in the first-layer filter gradient
    {"conv64_no_mfma", 0},             // 1: double-precision convolutions never on the matrix instruction
    {"pool64_no_tiles", 0},            // 1: max-pool backward in double never by tiles through LDS
    {"conv_no_first", 0},              // 1: never use the filter-gradient kernel for first layers (few input channels)
    {"conv_no_few", 0},                // 1: never use the kernel for products with at most four output channels
    {"conv_ws_min_units", 0},          // least number of units for the weights-stationary kernel; 0 = one per two SIMDs
    {"conv_ws_sliced_strided", 0},     // 1: sliced banks also for strided gathers (slower than the tiled kernel)
    {"conv_ws_wa", 0},                 // 1, 2, 4: force its channels-per-wavefront (in units of 32); 0 = choose
    {"conv_no_split", 0},              // 1: the tiled kernel never splits its reduction over workgroups
    {"conv_pix_multi", 1},             // the stride classes of a strided backward-data product share one launch where they can
    {"conv_force_direct", 0},          // 1: always use the direct (non-MFMA) convolution kernels
    {"conv_no_uniform_tap", 0},        // 1: disable the uniform-tap variant of the pixel-major kernel
    {"conv_wgrad_no_wide_rows", 0},    // 1: no 192-row filter-gradient tiles
};
}  // namespace

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_message, sizeof(g_message), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_message[0] = 0; }

int check_launch(const char* what) {
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(MCN_DEVICE_ERROR, "%s: %s", what, hipGetErrorString(e));
  }
  return MCN_SUCCESS;
}

namespace {
struct ProfileState {
  std::mutex mutex;
  std::atomic<bool> active{false};
  std::string pattern;
  std::vector<hipEvent_t> begin, end;
  size_t used = 0;
} g_profile;
}  // namespace

KernelTimer::KernelTimer(const char* kernel, hipStream_t s) : slot(-1), stream(s) {
  if (!g_profile.active.load(std::memory_order_relaxed)) return;
  std::lock_guard<std::mutex> lock(g_profile.mutex);
  if (!g_profile.active || std::strstr(kernel, g_profile.pattern.c_str()) == nullptr) return;
  if (g_profile.used == g_profile.begin.size()) {
    hipEvent_t b, e;
    if (hipEventCreate(&b) != hipSuccess || hipEventCreate(&e) != hipSuccess) return;
    g_profile.begin.push_back(b);
    g_profile.end.push_back(e);
  }
  slot = (int)g_profile.used++;
  (void)hipEventRecord(g_profile.begin[slot], stream);
}

KernelTimer::~KernelTimer() {
  if (slot < 0) return;
  std::lock_guard<std::mutex> lock(g_profile.mutex);
  (void)hipEventRecord(g_profile.end[slot], stream);
}

int tunable(const char* name, int fallback) {
  for (auto& t : g_tunables)
    if (std::strcmp(t.name, name) == 0) return t.value.load(std::memory_order_relaxed);
  return fallback;
}

namespace {
constexpr int kMaxBeside = 16;
std::atomic<void*> g_beside[kMaxBeside];
}  // namespace

bool stream_beside(hipStream_t s) {
  if (!s) return false;
  for (auto& slot : g_beside)
    if (slot.load(std::memory_order_relaxed) == (void*)s) return true;
  return false;
}

int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  return dev;
}

int device_compute_units() {
  static std::atomic<int> cached[kMaxDevices];  // 0 = not asked yet
  const int dev = current_device();
  if (dev < 0) return -1;
  if (dev < kMaxDevices) {
    const int have = cached[dev].load(std::memory_order_relaxed);
    if (have > 0) return have;
  }
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
    (void)hipGetLastError();
    return -1;
  }
  if (dev < kMaxDevices) cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

}  // namespace mcn

extern "C" {

const char* mcn_last_error_message(void) { return mcn::g_message; }

int mcn_stream_beside(mcn_stream_t stream, int on) {
  using namespace mcn;
  if (!stream) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_stream_beside: the null stream cannot be marked");
  // (not a hot path: marking and unmarking are serialised, so a stream holds at most one slot and unmarking frees it)
  static std::mutex mutex;
  std::lock_guard<std::mutex> lock(mutex);
  bool marked = false;
  for (auto& slot : g_beside)
    if (slot.load(std::memory_order_relaxed) == (void*)stream) {
      if (!on) slot.store(nullptr, std::memory_order_relaxed);  // (every slot that holds it)
      marked = true;
    }
  if (!on || marked) return MCN_SUCCESS;
  for (auto& slot : g_beside)
    if (slot.load(std::memory_order_relaxed) == nullptr) {
      slot.store((void*)stream, std::memory_order_relaxed);
      return MCN_SUCCESS;
    }
  return fail(MCN_UNSUPPORTED, "mcn_stream_beside: %d streams are marked already", kMaxBeside);
}

const char* mcn_error_name(int code) {
  switch (code) {
    case MCN_SUCCESS: return "success";
    case MCN_UNSUPPORTED: return "unsupported feature error";
    case MCN_DEVICE_ERROR: return "HIP error";
    case MCN_OUT_OF_MEMORY: return "out of memory error";
    case MCN_OUT_OF_GPU_MEMORY: return "out of GPU memory error";
    case MCN_ILLEGAL_ARGUMENT: return "illegal argument error";
    default: return "unknown error";
  }
}

int mcn_device_compute_units(void) { return mcn::device_compute_units(); }

int mcn_profile_begin(const char* kernel_name) {
  if (!kernel_name || !*kernel_name) return mcn::fail(MCN_ILLEGAL_ARGUMENT, "mcn_profile_begin: empty kernel name");
  std::lock_guard<std::mutex> lock(mcn::g_profile.mutex);
  mcn::g_profile.pattern = kernel_name;
  mcn::g_profile.used = 0;
  mcn::g_profile.active = true;
  return MCN_SUCCESS;
}

int mcn_profile_end(int* launches, double* total_ms) {
  std::lock_guard<std::mutex> lock(mcn::g_profile.mutex);
  mcn::g_profile.active = false;
  double total = 0.0;
  const size_t n = mcn::g_profile.used;
  if (n > 0 && hipEventSynchronize(mcn::g_profile.end[n - 1]) != hipSuccess)
    return mcn::fail(MCN_DEVICE_ERROR, "mcn_profile_end: event synchronisation failed");
  for (size_t i = 0; i < n; ++i) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, mcn::g_profile.begin[i], mcn::g_profile.end[i]) != hipSuccess)
      return mcn::fail(MCN_DEVICE_ERROR, "mcn_profile_end: event %zu was not recorded", i);
    total += ms;
  }
  if (launches) *launches = (int)n;
  if (total_ms) *total_ms = total;
  mcn::g_profile.used = 0;
  return MCN_SUCCESS;
}

int mcn_set_tunable(const char* name, int value) {
  if (!name) return mcn::fail(MCN_ILLEGAL_ARGUMENT, "mcn_set_tunable: null name");
  for (auto& t : mcn::g_tunables)
    if (std::strcmp(t.name, name) == 0) {
      t.value.store(value, std::memory_order_relaxed);
      return MCN_SUCCESS;
    }
  return mcn::fail(MCN_ILLEGAL_ARGUMENT, "mcn_set_tunable: unknown tunable '%s'", name);
}

int mcn_get_tunable(const char* name, int* value) {
  if (!name || !value) return mcn::fail(MCN_ILLEGAL_ARGUMENT, "mcn_get_tunable: null argument");
  for (auto& t : mcn::g_tunables)
    if (std::strcmp(t.name, name) == 0) {
      *value = t.value.load(std::memory_order_relaxed);
      return MCN_SUCCESS;
    }
  return mcn::fail(MCN_ILLEGAL_ARGUMENT, "mcn_get_tunable: unknown tunable '%s'", name);
}

}  // extern "C"
