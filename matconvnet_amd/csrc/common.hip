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
    {"conv_wgrad_wide_rows_exact", 1}, // 192-row filter-gradient tiles for volumes they cover exactly and 128-row tiles do not
    {"conv_pix_direct", 1},            // tiled kernel: the loads of a step go straight into LDS, a few at a time between the MFMAs (0: through registers)
    {"conv_wgrad_direct", 1},          // filter gradient: the loads of a step go straight into LDS, a few at a time between the MFMAs (0: through registers)
    {"conv_no_sb", 0},                 // 1: the streamed-bank kernel is not used (banks too large for LDS go to the tiled kernel)
    {"conv_sb_split", 0},              // 0: the streamed-bank kernel leaves products whose reduction it would split to the tiled kernel
                                       // (on their own, warm, the split products win 8-11% at 32 images; inside ResNet-50 the step loses 0.17 ms)
    {"conv_sb_slab", 32},              // reduction rows per slab of the bank in LDS (32 or 64) of the streamed-bank kernel
    {"conv_sb_occupancy", 2},          // wavefronts per SIMD the 128-channel streamed-bank kernel's registers are cut for (2 or 3)
    {"conv_sb_fill", 2},               // workgroups per compute unit below which the streamed-bank kernel splits the reduction
    {"conv_sb_tail", 1},               // streamed-bank kernel: the tiles of a partly filled last round get a launch of their own that splits their reduction
    {"conv_sb_tail_slots", 0},         // resident workgroups per compute unit that plan assumes (0: the instantiation's own)
    {"conv_sb_tail_min_pairs", 2},     // least pairs of slabs per split of a tail tile
    {"conv_sb_tail_max_splits", 16},   // most splits of a tail tile
    {"conv_sb_min_pairs", 6},          // least pairs of 32-row slabs per split of the streamed-bank kernel
    {"pool_lds_bytes", 16 * 1024},     // LDS tile budget of the pooling-backward kernels
    {"pool_no_pairs", 0},              // 1: max pooling skips the kernel for 3x3 windows at stride 2, padding 1
    {"pool_pairs_per_cu", 0},          // its persistent workgroups per compute unit (0: as many as fit)
    {"pool_pairs_cols", 0},            // n > 0: its tiles are n output columns wide (0: chosen)
    {"pool_pairs_stages", 3},          // 2 or 3 stages of a tile's operands in LDS (1 or 2 tiles in flight per workgroup)
    {"pool_pairs_static", 0},          // 1: the workgroups of a compute unit take equal shares of its tiles
    {"pool_no_stream", 0},             // 1: max pooling skips the streaming kernel
    {"pool_walk", 3},                  // streaming kernel's tile order: 0 round-robin, 1 contiguous runs, 2 round-robin per XCD eighth, 3 planes round-robin over XCDs
    {"bnorm_walk", 1},                 // order of batch normalisation's workgroups: 1 by plane address (image-major), 0 channel-major and XCD by XCD, 2 by plane address and XCD by XCD
    {"bnorm_sums_scalar", 0},          // 1: the summing pass of batch-norm backward (moments from the batch) loads 4 bytes per lane, four in flight
    {"pool_no_tiles", 0},              // 1: average pooling over windows that tile the plane skips its streaming kernel
    {"pool_threads", 256},             // threads per workgroup of the streaming kernel (256; 512 and 1024 for 3x3 / 2 windows)
    {"pool_blocks_per_cu", 3},         // persistent workgroups per compute unit of the streaming kernel
    {"pool_forward_threads_k", 2048},  // threads (in 1024s) the four-rows-per-thread forward kernel aims at
    {"pool_force_gather", 0},          // 1: skip the ordered-pass kernel, use the general tiled gather
    {"bnorm_block_elems", 4096},       // minimum elements a bnorm reduction block should own
    {"bnorm_one_launch_elems", 8192},  // channels of at most this many elements (and >= 128 of them): sums and apply in one launch
    {"bnorm_reverse_apply", 1},        // second bnorm pass walks planes in reverse (cache reuse)
    {"conv_no_ws", 0},                 // 1: never use the weights-stationary kernel
    {"conv_first_per_cu", 0},          // > 0: workgroups per compute unit of the first-layer filter gradient (else by its registers)
    {"conv_first_max_wg", 0},          // > 0: at most this many workgroups in the first-layer filter gradient
    {"conv64_no_mfma", 0},             // 1: double-precision convolutions never on the matrix instruction
    {"pool64_tile_kb", 40},
    {"pool64_walk_per_cu", 0},
    {"pool64_no_tiles", 0},            // 1: max-pool backward in double never by tiles through LDS
    {"conv_no_first", 0},              // 1: never use the filter-gradient kernel for first layers (few input channels)
    {"conv_first_no_vec", 0},          // 1: the first-layer filter gradient stages its tiles 4 bytes per lane always
    {"conv_no_few", 0},                // 1: never use the kernel for products with at most four output channels
    {"conv_ws_min_units", 0},          // least number of units for the weights-stationary kernel; 0 = one per two SIMDs
    {"conv_ws_max_slices", 8},         // most slices of output channels its bank may be cut into (1: whole banks only)
    {"conv_ws_sliced_strided", 0},     // 1: sliced banks also for strided gathers (slower than the tiled kernel)
    {"conv_ws_fill", 4},               // units per SIMD from which its wide units are considered
    {"conv_ws_wa", 0},                 // 1, 2, 4: force its channels-per-wavefront (in units of 32); 0 = choose
    {"conv_no_split", 0},              // 1: the tiled kernel never splits its reduction over workgroups
    {"conv_split_max_blocks", 512},    // ... it splits when the unsplit launch has at most this many workgroups,
    {"conv_split_most", 16},           // into at most this many parts (the count is chosen by a model of the time),
    {"conv_split_min_steps", 12},      // with at least this many 16-row steps left to each
    {"conv_split_force", 0},           // n > 0: exactly n splits (experiments)
    {"conv_wgrad_beside_kb", 84},      // local memory a filter-gradient launch asks for on a stream marked by mcn_stream_beside
    {"conv_ws_deep_copy", 1},
    {"conv_wgrad_deep", 1},            // filter gradients of at most one workgroup per CU load two steps ahead (three LDS buffers)
    {"conv_pix_multi", 1},             // the stride classes of a strided backward-data product share one launch where they can
    {"conv_pix_multi_tiles", 4096},    // ... up to this many tiles in all (larger layers: a launch per class)
    {"conv_pack_tiled", 1},            // forward banks are packed tile by tile through LDS (0: element by element)
    {"conv_no_fc_view", 0},            // 1: fully-connected layers are not recast as 1x1 layers
    {"conv_force_direct", 0},          // 1: always use the direct (non-MFMA) convolution kernels
    {"conv_pix_tile", 0},              // force a tile shape of the pixel-major MFMA kernel (0 = automatic)
    {"conv_no_uniform_tap", 0},        // 1: disable the uniform-tap variant of the pixel-major kernel
    {"conv_wgrad_no_wide_rows", 0},    // 1: no 192-row filter-gradient tiles
    {"conv_wgrad_no_small_rule", 0},   // 1: always two filter-gradient workgroups per CU
    {"conv_wgrad_blocks", 0},          // target workgroups for filter-gradient split (0 = 2 per CU)
    {"conv_bias_blocks", 0},           // target workgroups for the bias-gradient reduction
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
