// Convolution entry points: validation, dispatch between the MFMA implicit-GEMM kernels and the direct
// kernels, and the bias-gradient reduction.
#include "conv_common.hpp"

#include <cstring>
#include <vector>

#include <algorithm>

namespace mcn {

int conv_setup(const mcn_conv_geom* g, const char* who, ConvP* p) {
  if (!g) return fail(MCN_ILLEGAL_ARGUMENT, "%s: null geometry", who);
  if (g->H < 0 || g->W < 0 || g->C < 0 || g->N < 0) return fail(MCN_ILLEGAL_ARGUMENT, "%s: negative tensor extent", who);
  if (g->strideY < 1 || g->strideX < 1)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: at least one element of STRIDE is smaller than one", who);
  if (g->padTop < 0 || g->padBottom < 0 || g->padLeft < 0 || g->padRight < 0)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: an element of PAD is negative", who);
  if (g->dilateY < 1 || g->dilateX < 1) return fail(MCN_ILLEGAL_ARGUMENT, "%s: an element of DILATE is less than one", who);
  if (g->FH < 1 || g->FW < 1 || g->FC < 1 || g->K < 1) return fail(MCN_ILLEGAL_ARGUMENT, "%s: a dimension of FILTERS is void", who);
  const int extY = (g->FH - 1) * g->dilateY + 1, extX = (g->FW - 1) * g->dilateX + 1;
  if (g->H + g->padTop + g->padBottom < extY || g->W + g->padLeft + g->padRight < extX)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: FILTERS are larger than the DATA (including padding)", who);
  const int groups = g->C / g->FC;
  if (groups * g->FC != g->C) return fail(MCN_ILLEGAL_ARGUMENT, "%s: the FILTERS depth does not divide the DATA depth", who);
  if (groups < 1 || g->K % groups != 0)
    return fail(MCN_ILLEGAL_ARGUMENT, "%s: the number of filter groups does not divide the number of filters", who);
  p->H = g->H; p->W = g->W; p->C = g->C; p->N = g->N;
  p->FH = g->FH; p->FW = g->FW; p->FC = g->FC; p->K = g->K;
  p->sy = g->strideY; p->sx = g->strideX; p->pt = g->padTop; p->pl = g->padLeft;
  p->dy = g->dilateY; p->dx = g->dilateX;
  p->outH = (g->H + g->padTop + g->padBottom - extY) / g->strideY + 1;
  p->outW = (g->W + g->padLeft + g->padRight - extX) / g->strideX + 1;
  p->groups = groups;
  p->Kg = g->K / groups;
  const long long lim = 1ll << 31;
  if ((long long)g->H * g->W * g->C >= lim || (long long)p->outH * p->outW * g->K >= lim ||
      (long long)g->FH * g->FW * g->FC * g->K >= lim)
    return fail(MCN_UNSUPPORTED, "%s: an image or the filter bank exceeds 2^31 elements", who);
  return MCN_SUCCESS;
}

namespace {

// ---- bias gradient: db[k] = sum_{n,p} dy[p,k,n].
// Stage 1: grid (k, image group); lanes stream planes with 16-byte loads, fp32 per plane per lane, fp64
// above, wavefront shuffle reduction + LDS across the four wavefronts.  Stage 2: one lane per filter adds
// the image-group partials in a fixed order.
template <bool VEC4>
__global__ __launch_bounds__(256) void conv_bias_partial(double* __restrict__ partials,
                                                         const float* __restrict__ dy, int P, int K, int N,
                                                         int groups) {
  __shared__ double lds[4];
  const int logical = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int k = logical / groups, grp = logical - k * groups;
  const int n0 = (int)(((long long)N * grp) / groups), n1 = (int)(((long long)N * (grp + 1)) / groups);
  double acc = 0.0;
  for (int n = n0; n < n1; ++n) {
    const float* src = dy + (size_t)P * (k + (size_t)K * n);
    float s = 0.f;
    if (VEC4) {
      const float4* s4 = (const float4*)src;
      for (int i = threadIdx.x; i < P / 4; i += 256) {
        const float4 v = s4[i];
        s += (v.x + v.y) + (v.z + v.w);
      }
    } else {
      for (int i = threadIdx.x; i < P; i += 256) s += src[i];
    }
    acc += (double)s;
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) partials[(size_t)k * groups + grp] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

__global__ __launch_bounds__(256) void conv_bias_finish(float* __restrict__ db, const double* __restrict__ partials,
                                                        int K, int groups) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k >= K) return;
  double s = 0.0;
  for (int g = 0; g < groups; ++g) s += partials[(size_t)k * groups + g];
  db[k] = (float)s;
}

int bias_groups(const ConvP& p) {
  const int target = 2048;
  const int P = p.outH * p.outW;
  const int perBlock = std::max(1, 4096 / std::max(P, 1));  // at least ~4096 elements per workgroup
  const int maxGroups = std::max(1, (p.N + perBlock - 1) / perBlock);
  return std::max(1, std::min(maxGroups, (target + p.K - 1) / p.K));
}

}  // namespace
}  // namespace mcn

using namespace mcn;

extern "C" {

int mcn_conv_output_size(const mcn_conv_geom* g, int* outH, int* outW) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_output_size", &p);
  if (rc) return rc;
  if (outH) *outH = p.outH;
  if (outW) *outW = p.outW;
  return MCN_SUCCESS;
}

size_t mcn_conv_workspace_bytes(const mcn_conv_geom* g, int product) {
  ConvP p;
  if (conv_setup(g, "mcn_conv_workspace_bytes", &p)) return 0;
  if (p.N == 0) return 0;
  if (product == MCN_CONV_BACKWARD_BIAS) return (size_t)p.K * bias_groups(p) * sizeof(double);
  size_t bytes = conv_mfma_workspace_bytes(p, product);
  if (product == MCN_CONV_BACKWARD_FILTER && conv_first_backward_filter_supported(p)) bytes = std::max(bytes, conv_first_workspace_bytes(p));
  return bytes;
}

int mcn_conv_forward(mcn_stream_t stream, const mcn_conv_geom* g, float* y, float outMult, const float* x,
                     float inMult, const float* filters, const float* bias, void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_forward", &p);
  if (rc) return rc;
  if ((size_t)p.outH * p.outW * p.K * p.N == 0) return MCN_SUCCESS;
  if (!y || !x || !filters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_forward: null tensor");
  if (!tunable("conv_force_direct", 0) && outMult == 0.f && inMult == 1.f && conv_first_forward_supported(p))
    return conv_first_forward(as_stream(stream), p, y, x, filters, bias);
  if (!tunable("conv_force_direct", 0) && conv_mfma_forward_supported(p))
    return conv_forward_mfma(as_stream(stream), p, y, outMult, x, inMult, filters, bias, workspace, workspaceBytes);
  return conv_forward_direct(as_stream(stream), p, y, outMult, x, inMult, filters, bias);
}

int mcn_conv_backward_data_acc(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, float derInputMult,
                               const float* filters, const float* derOutput, void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_data", &p);
  if (rc) return rc;
  if ((size_t)p.H * p.W * p.C * p.N == 0) return MCN_SUCCESS;
  if (!derInput || !filters || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_data: null tensor");
  if (!tunable("conv_force_direct", 0) && derInputMult == 0.f && conv_first_backward_data_supported(p))
    return conv_first_backward_data(as_stream(stream), p, derInput, filters, derOutput);
  if (!tunable("conv_force_direct", 0) && conv_mfma_backward_data_supported(p))
    return conv_backward_data_mfma(as_stream(stream), p, derInput, derInputMult, filters, derOutput, workspace, workspaceBytes);
  return conv_backward_data_direct(as_stream(stream), p, derInput, derInputMult, filters, derOutput);
}

namespace {
// the three uses of a packed-ahead buffer share the walk over a product's banks
int walk_packed(hipStream_t s, const ConvP& p, int product, const float* filters, PackCtx* pk) {
  float* dummy = const_cast<float*>(filters);  // (no tensor is touched when planning or packing)
  if (product == MCN_CONV_FORWARD) {
    if (!conv_mfma_forward_supported(p) || tunable("conv_force_direct", 0)) return MCN_SUCCESS;
    return conv_forward_mfma(s, p, dummy, 0.f, dummy, 1.f, filters, nullptr, nullptr, 0, pk);
  }
  if (product == MCN_CONV_BACKWARD_DATA) {
    if (!conv_mfma_backward_data_supported(p) || tunable("conv_force_direct", 0)) return MCN_SUCCESS;
    return conv_backward_data_mfma(s, p, dummy, 0.f, filters, dummy, nullptr, 0, pk);
  }
  return fail(MCN_ILLEGAL_ARGUMENT, "packed filters exist for the forward and the backward-data product only");
}
static_assert(sizeof(PackJob) <= sizeof(mcn_conv_pack_job), "mcn_conv_pack_job must hold a PackJob");
}  // namespace

size_t mcn_conv_packed_bytes(const mcn_conv_geom* g, int product) {
  ConvP p;
  if (conv_setup(g, "mcn_conv_packed_bytes", &p) || p.N == 0) return 0;
  PackCtx pk = {PackCtx::kPlan, nullptr, 0, 0, nullptr};
  if (walk_packed(nullptr, p, product, nullptr, &pk)) return 0;
  return pk.offset;
}

int mcn_conv_pack_filters(mcn_stream_t stream, const mcn_conv_geom* g, int product, const float* filters, void* packed,
                          size_t packedBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_pack_filters", &p);
  if (rc) return rc;
  if (p.N == 0) return MCN_SUCCESS;
  if (!filters || (!packed && packedBytes)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_filters: null argument");
  if (!aligned16(packed)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_filters: the buffer must be 16-byte aligned");
  PackCtx pk = {PackCtx::kPack, (char*)packed, packedBytes, 0, nullptr};
  return walk_packed(as_stream(stream), p, product, filters, &pk);
}

int mcn_conv_pack_plan(const mcn_conv_geom* g, int product, const float* filters, void* packed, size_t packedBytes,
                       mcn_conv_pack_job* jobs, int maxJobs, int* nJobs) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_pack_plan", &p);
  if (rc) return rc;
  if (!nJobs) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_plan: null argument");
  *nJobs = 0;
  if (p.N == 0) return MCN_SUCCESS;
  std::vector<PackJob> found;
  PackCtx pk = {PackCtx::kPlan, (char*)packed, packedBytes, 0, &found};
  if ((rc = walk_packed(nullptr, p, product, filters, &pk))) return rc;
  if (pk.offset > packedBytes) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_plan: packed filter buffer too small");
  if ((int)found.size() > maxJobs) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_plan: more than %d jobs", maxJobs);
  for (size_t i = 0; i < found.size(); ++i) {
    std::memset(&jobs[i], 0, sizeof(jobs[i]));
    std::memcpy(&jobs[i], &found[i], sizeof(PackJob));
  }
  *nJobs = (int)found.size();
  return MCN_SUCCESS;
}

unsigned mcn_conv_pack_layout(mcn_conv_pack_job* jobs, int nJobs) {
  unsigned at = 0;
  for (int i = 0; i < nJobs; ++i) {
    PackJob j;
    std::memcpy(&j, &jobs[i], sizeof(PackJob));
    j.firstBlock = at;
    at += j.blocks;
    std::memcpy(&jobs[i], &j, sizeof(PackJob));
  }
  return at;
}

int mcn_conv_pack_batch(mcn_stream_t stream, const mcn_conv_pack_job* deviceJobs, int nJobs, unsigned totalBlocks) {
  if (nJobs > 0 && !deviceJobs) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_pack_batch: null argument");
  static_assert(sizeof(mcn_conv_pack_job) == sizeof(PackJob), "a device array of mcn_conv_pack_job is read as PackJob[]");
  return conv_pack_batch(as_stream(stream), (const PackJob*)deviceJobs, nJobs, totalBlocks);
}

int mcn_conv_forward_packed(mcn_stream_t stream, const mcn_conv_geom* g, float* y, float outMult, const float* x,
                            float inMult, const float* filters, const void* packed, size_t packedBytes, const float* bias,
                            void* workspace, size_t workspaceBytes) {
  if (!packed) return mcn_conv_forward(stream, g, y, outMult, x, inMult, filters, bias, workspace, workspaceBytes);
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_forward", &p);
  if (rc) return rc;
  if ((size_t)p.outH * p.outW * p.K * p.N == 0) return MCN_SUCCESS;
  if (!y || !x || !filters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_forward: null tensor");
  if (!tunable("conv_force_direct", 0) && outMult == 0.f && inMult == 1.f && conv_first_forward_supported(p))
    return conv_first_forward(as_stream(stream), p, y, x, filters, bias);  // (reads the bank as it is stored)
  if (!tunable("conv_force_direct", 0) && conv_mfma_forward_supported(p)) {
    PackCtx pk = {PackCtx::kUse, (char*)const_cast<void*>(packed), packedBytes, 0, nullptr};
    return conv_forward_mfma(as_stream(stream), p, y, outMult, x, inMult, filters, bias, workspace, workspaceBytes, &pk);
  }
  return conv_forward_direct(as_stream(stream), p, y, outMult, x, inMult, filters, bias);
}

int mcn_conv_forward_sums_groups(const mcn_conv_geom* g) {
  ConvP p;
  if (conv_setup(g, "mcn_conv_forward_sums_groups", &p) || (size_t)p.outH * p.outW * p.K * p.N == 0) return 0;
  if (tunable("conv_force_direct", 0) || !conv_mfma_forward_supported(p)) return 0;
  int groups = 0;
  float* dummy = nullptr;  // (nothing is touched when planning)
  if (conv_forward_mfma(nullptr, p, dummy, 0.f, dummy, 1.f, dummy, nullptr, nullptr, 0, nullptr, nullptr, 0, &groups)) return 0;
  return groups;
}

int mcn_conv_forward_sums(mcn_stream_t stream, const mcn_conv_geom* g, float* y, const float* x, const float* filters,
                          const void* packed, size_t packedBytes, double* sums, size_t sumsBytes, void* workspace,
                          size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_forward_sums", &p);
  if (rc) return rc;
  if (!y || !x || !filters || !sums) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_forward_sums: null tensor");
  const int groups = mcn_conv_forward_sums_groups(g);
  if (groups <= 0) return fail(MCN_UNSUPPORTED, "mcn_conv_forward_sums: this geometry has no such form (ask mcn_conv_forward_sums_groups)");
  if (sumsBytes < (size_t)p.K * groups * 2 * sizeof(double))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_forward_sums: the buffer of partial sums is too small");
  if (packed) {
    PackCtx pk = {PackCtx::kUse, (char*)const_cast<void*>(packed), packedBytes, 0, nullptr};
    return conv_forward_mfma(as_stream(stream), p, y, 0.f, x, 1.f, filters, nullptr, workspace, workspaceBytes, &pk, sums, groups);
  }
  return conv_forward_mfma(as_stream(stream), p, y, 0.f, x, 1.f, filters, nullptr, workspace, workspaceBytes, nullptr, sums, groups);
}

int mcn_conv_backward_data_packed(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, float derInputMult,
                                  const float* filters, const void* packed, size_t packedBytes, const float* derOutput,
                                  void* workspace, size_t workspaceBytes) {
  if (!packed)
    return mcn_conv_backward_data_acc(stream, g, derInput, derInputMult, filters, derOutput, workspace, workspaceBytes);
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_data", &p);
  if (rc) return rc;
  if ((size_t)p.H * p.W * p.C * p.N == 0) return MCN_SUCCESS;
  if (!derInput || !filters || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_data: null tensor");
  if (!tunable("conv_force_direct", 0) && derInputMult == 0.f && conv_first_backward_data_supported(p))
    return conv_first_backward_data(as_stream(stream), p, derInput, filters, derOutput);  // (reads the bank as it is stored)
  if (!tunable("conv_force_direct", 0) && conv_mfma_backward_data_supported(p)) {
    PackCtx pk = {PackCtx::kUse, (char*)const_cast<void*>(packed), packedBytes, 0, nullptr};
    return conv_backward_data_mfma(as_stream(stream), p, derInput, derInputMult, filters, derOutput, workspace,
                                   workspaceBytes, &pk);
  }
  return conv_backward_data_direct(as_stream(stream), p, derInput, derInputMult, filters, derOutput);
}

int mcn_conv_backward_data_masked_add_supported(const mcn_conv_geom* g) {
  ConvP p;
  if (conv_setup(g, "mcn_conv_backward_data_masked_add_supported", &p) || (size_t)p.H * p.W * p.C * p.N == 0) return 0;
  if (tunable("conv_force_direct", 0) || !conv_mfma_backward_data_supported(p)) return 0;
  int ok = 0;
  float* none = nullptr;  // (nothing is touched when planning)
  if (conv_backward_data_mfma(nullptr, p, none, 0.f, none, none, nullptr, 0, nullptr, nullptr, nullptr, &ok)) return 0;
  return ok;
}

int mcn_conv_backward_data_masked_add(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, const float* filters,
                                      const void* packed, size_t packedBytes, const float* derOutput, const float* addend,
                                      const unsigned* maskBits, void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_data_masked_add", &p);
  if (rc) return rc;
  if ((size_t)p.H * p.W * p.C * p.N == 0) return MCN_SUCCESS;
  if (!derInput || !filters || !derOutput || !addend || !maskBits)
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_data_masked_add: null tensor");
  if (!mcn_conv_backward_data_masked_add_supported(g))
    return fail(MCN_UNSUPPORTED, "mcn_conv_backward_data_masked_add: this geometry has no such form (ask "
                "mcn_conv_backward_data_masked_add_supported)");
  if (packed) {
    PackCtx pk = {PackCtx::kUse, (char*)const_cast<void*>(packed), packedBytes, 0, nullptr};
    return conv_backward_data_mfma(as_stream(stream), p, derInput, 0.f, filters, derOutput, workspace, workspaceBytes, &pk,
                                   addend, maskBits);
  }
  return conv_backward_data_mfma(as_stream(stream), p, derInput, 0.f, filters, derOutput, workspace, workspaceBytes, nullptr,
                                 addend, maskBits);
}

int mcn_conv_backward_data(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, const float* filters,
                           const float* derOutput, void* workspace, size_t workspaceBytes) {
  return mcn_conv_backward_data_acc(stream, g, derInput, 0.f, filters, derOutput, workspace, workspaceBytes);
}

int mcn_conv_backward_filter(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters, const float* x,
                             const float* derOutput, void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_filter", &p);
  if (rc) return rc;
  if (!derFilters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter: null tensor");
  const size_t nf = (size_t)p.FH * p.FW * p.FC * p.K;
  if ((size_t)p.outH * p.outW * p.N == 0) return mcn_fill(stream, derFilters, 0.f, nf);
  if (!x || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter: null tensor");
  if (!tunable("conv_force_direct", 0) && conv_first_backward_filter_supported(p))
    return conv_first_backward_filter(as_stream(stream), p, derFilters, nullptr, x, derOutput, workspace, workspaceBytes);
  if (!tunable("conv_force_direct", 0) && conv_mfma_backward_filter_supported(p))
    return conv_backward_filter_mfma(as_stream(stream), p, derFilters, x, derOutput, workspace, workspaceBytes);
  return conv_backward_filter_direct(as_stream(stream), p, derFilters, x, derOutput);
}

namespace {
static_assert(sizeof(ReduceJob) == sizeof(mcn_conv_reduce_job), "a device array of mcn_conv_reduce_job is read as ReduceJob[]");
bool deferred_available(const ConvP& p) {
  // (first layers have a kernel of their own, which sums its partial banks itself: no deferred form)
  return !tunable("conv_force_direct", 0) && !conv_first_backward_filter_supported(p) && conv_mfma_backward_filter_supported(p) &&
         (size_t)p.outH * p.outW * p.N != 0;
}
}  // namespace

size_t mcn_conv_backward_filter_partial_bytes(const mcn_conv_geom* g) {
  ConvP p;
  if (conv_setup(g, "mcn_conv_backward_filter_partial_bytes", &p) || !deferred_available(p)) return 0;
  ReduceCtx ctx = {nullptr, 0, 0, nullptr, false};
  float* dummy = nullptr;
  if (conv_backward_filter_mfma(nullptr, p, dummy, dummy, dummy, nullptr, 0, &ctx)) return 0;
  return ctx.offset;
}

int mcn_conv_backward_filter_plan(const mcn_conv_geom* g, float* derFilters, void* partials, size_t partialBytes,
                                  mcn_conv_reduce_job* jobs, int maxJobs, int* nJobs) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_filter_plan", &p);
  if (rc) return rc;
  if (!nJobs || !derFilters) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_plan: null argument");
  *nJobs = 0;
  if (!deferred_available(p)) return fail(MCN_UNSUPPORTED, "mcn_conv_backward_filter_plan: this geometry has no deferred sum");
  std::vector<ReduceJob> found;
  ReduceCtx ctx = {(char*)partials, partialBytes, 0, &found, false};
  if ((rc = conv_backward_filter_mfma(nullptr, p, derFilters, derFilters, derFilters, nullptr, 0, &ctx))) return rc;
  if (ctx.offset > partialBytes) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_plan: buffer of partial banks too small");
  if ((int)found.size() > maxJobs) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_plan: more than %d jobs", maxJobs);
  for (size_t i = 0; i < found.size(); ++i) std::memcpy(&jobs[i], &found[i], sizeof(ReduceJob));
  *nJobs = (int)found.size();
  return MCN_SUCCESS;
}

int mcn_conv_backward_filter_partial(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters, const float* x,
                                     const float* derOutput, void* partials, size_t partialBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_filter_partial", &p);
  if (rc) return rc;
  if (!derFilters || !x || !derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_partial: null tensor");
  if (!deferred_available(p)) return fail(MCN_UNSUPPORTED, "mcn_conv_backward_filter_partial: this geometry has no deferred sum");
  if (!aligned16(partials)) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_partial: the buffer must be 16-byte aligned");
  ReduceCtx ctx = {(char*)partials, partialBytes, 0, nullptr, true};
  return conv_backward_filter_mfma(as_stream(stream), p, derFilters, x, derOutput, nullptr, 0, &ctx);
}

unsigned mcn_conv_reduce_layout(mcn_conv_reduce_job* jobs, int nJobs) {
  unsigned at = 0;
  for (int i = 0; i < nJobs; ++i) {
    ReduceJob j;
    std::memcpy(&j, &jobs[i], sizeof(ReduceJob));
    j.firstBlock = at;
    at += j.blocks;
    std::memcpy(&jobs[i], &j, sizeof(ReduceJob));
  }
  return at;
}

int mcn_conv_reduce_batch(mcn_stream_t stream, const mcn_conv_reduce_job* deviceJobs, int nJobs, unsigned totalBlocks) {
  if (nJobs > 0 && !deviceJobs) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_reduce_batch: null argument");
  return conv_reduce_batch(as_stream(stream), (const ReduceJob*)deviceJobs, nJobs, totalBlocks);
}

int mcn_conv_backward_filter_bias(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters, float* derBias,
                                  const float* x, const float* derOutput, void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_filter_bias", &p);
  if (rc) return rc;
  if (!derFilters || !derBias) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_filter_bias: null tensor");
  // a first layer: one pass gives both (the bias gradient is the column of the product that multiplies a row of ones)
  if ((size_t)p.outH * p.outW * p.N != 0 && x && derOutput && !tunable("conv_force_direct", 0) &&
      conv_first_backward_filter_supported(p))
    return conv_first_backward_filter(as_stream(stream), p, derFilters, derBias, x, derOutput, workspace, workspaceBytes);
  // otherwise the two products one after the other, through the same workspace
  rc = mcn_conv_backward_filter(stream, g, derFilters, x, derOutput, workspace, workspaceBytes);
  if (rc) return rc;
  return mcn_conv_backward_bias(stream, g, derBias, derOutput, workspace, workspaceBytes);
}

int mcn_conv_backward_bias(mcn_stream_t stream, const mcn_conv_geom* g, float* derBias, const float* derOutput,
                           void* workspace, size_t workspaceBytes) {
  ConvP p;
  int rc = conv_setup(g, "mcn_conv_backward_bias", &p);
  if (rc) return rc;
  if (!derBias) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_bias: null tensor");
  const int P = p.outH * p.outW;
  if ((size_t)P * p.N == 0) return mcn_fill(stream, derBias, 0.f, (size_t)p.K);
  if (!derOutput) return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_bias: null tensor");
  const int groups = bias_groups(p);
  if (!workspace || workspaceBytes < (size_t)p.K * groups * sizeof(double))
    return fail(MCN_ILLEGAL_ARGUMENT, "mcn_conv_backward_bias: workspace too small");
  double* partials = (double*)workspace;
  hipStream_t s = as_stream(stream);
  const bool vec = (P % 4 == 0) && aligned16(derOutput);
  const dim3 grid((unsigned)(p.K * groups)), block(256);
  KernelTimer timer("conv_bias_partial", s);
  if (vec) hipLaunchKernelGGL(conv_bias_partial<true>, grid, block, 0, s, partials, derOutput, P, p.K, p.N, groups);
  else hipLaunchKernelGGL(conv_bias_partial<false>, grid, block, 0, s, partials, derOutput, P, p.K, p.N, groups);
  if ((rc = check_launch("mcn_conv_backward_bias(partial)"))) return rc;
  hipLaunchKernelGGL(conv_bias_finish, dim3((unsigned)((p.K + 255) / 256)), block, 0, s, derBias, partials, p.K, groups);
  return check_launch("mcn_conv_backward_bias");
}

}  // extern "C"
