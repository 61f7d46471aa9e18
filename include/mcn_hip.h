/*
 * mcn_hip.h -- C ABI of the MI355X (gfx950) back-end for MatConvNet's convolution, batch-normalisation
 * and pooling operators.
 *
 * This is the layer the reference's device structs call into: where MatConvNet's
 * `ConvolutionBackward<VLDT_GPU,T>`, `BatchNormBackward<VLDT_GPU,T>` and `PoolingBackward<VLDT_GPU,T>`
 * launch CUDA kernels / cuBLAS / cuDNN, the replacement `VLDT_GPU` branch calls the functions below.
 *
 * Conventions
 *   - every tensor is fp32, MATLAB column-major H x W x C x N: element (h,w,c,n) at
 *     h + H*(w + W*(c + C*n)); filters FH x FW x FC x K likewise (bits/nnpooling.cu:131, nnconv.cu:132);
 *   - all pointers are DEVICE pointers on the current HIP device; `stream` is a hipStream_t passed as
 *     void* (NULL = the default stream); calls only enqueue work, they never synchronise;
 *   - scratch memory is supplied by the caller (the role of vl::Context::getWorkspace,
 *     bits/data.cu:395-404): ask mcn_*_workspace_bytes, pass a buffer of at least that many bytes,
 *     256-byte aligned; contents need not be preserved between calls;
 *   - return value: 0 on success, otherwise a code numerically equal to the matching vl::ErrorCode
 *     (bits/data.hpp:38-52); mcn_last_error_message() gives the text for the calling thread;
 *   - shapes are validated on the host before any launch; nothing is launched on error.
 */
#ifndef MCN_HIP_H
#define MCN_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define MCN_API __attribute__((visibility("default")))
#else
#define MCN_API
#endif

typedef void* mcn_stream_t;

/* numerically equal to vl::ErrorCode (bits/data.hpp:38-52) */
enum {
  MCN_SUCCESS = 0,
  MCN_UNSUPPORTED = 1,
  MCN_DEVICE_ERROR = 2, /* VLE_Cuda: a HIP runtime call or launch failed */
  MCN_OUT_OF_MEMORY = 5,
  MCN_OUT_OF_GPU_MEMORY = 6,
  MCN_ILLEGAL_ARGUMENT = 7,
  MCN_UNKNOWN = 8
};

/* vl::nn::Convolution's public members (bits/nnconv.hpp:43-51) plus the tensor extents the MEX driver
   checks (vl_nnconv.cu:269-342).  groups = C / FC; K must be a multiple of groups. */
typedef struct mcn_conv_geom {
  int H, W, C, N;    /* input x */
  int FH, FW, FC, K; /* filters */
  int strideY, strideX;
  int padTop, padBottom, padLeft, padRight;
  int dilateY, dilateX;
} mcn_conv_geom;

/* vl::nn::Pooling's public members (bits/nnpooling.hpp:39-48) plus the input extents. */
typedef struct mcn_pool_geom {
  int H, W, C, N;
  int poolH, poolW;
  int strideY, strideX;
  int padTop, padBottom, padLeft, padRight;
  int method; /* 0 = vl::nn::Pooling::Max, 1 = Average */
} mcn_pool_geom;

enum { MCN_POOL_MAX = 0, MCN_POOL_AVERAGE = 1 };

/* which convolution product a workspace query is for */
enum { MCN_CONV_FORWARD = 0, MCN_CONV_BACKWARD_DATA = 1, MCN_CONV_BACKWARD_FILTER = 2, MCN_CONV_BACKWARD_BIAS = 3 };

/* ------------------------------------------------------------------------------------------------
 * library
 * ---------------------------------------------------------------------------------------------- */

/* Text of the last error raised on the calling thread (never NULL).  Replaces the message path of
   vl::Context::setError / getLastErrorMessage (bits/data.cu:332-377) below the operator layer. */
MCN_API const char* mcn_last_error_message(void);

/* Generic name of an error code; same strings as vl::getErrorMessage (bits/data.cu:83-96). */
MCN_API const char* mcn_error_name(int code);

/* Compute units of the current device (for sizing grids / reporting); <0 on error. */
MCN_API int mcn_device_compute_units(void);

/* Name/value knobs for experiments (tile budgets, split factors).  Unknown names are rejected.
   Not part of the reference interface. */
MCN_API int mcn_set_tunable(const char* name, int value);
MCN_API int mcn_get_tunable(const char* name, int* value);

/* Marks a stream (not the null stream) as one whose launches run BESIDE another stream's kernels -- a caller that puts
   the filter gradients of a backward pass on a second stream, next to the input gradients on the first.  Launches on a
   marked stream ask for so much local memory that a compute unit holds one of their workgroups at a time: the kernels
   on the other stream, which the rest of the pass waits for, keep most of every compute unit (ResNet-50 training step
   at 32 images with the filter gradients on a second stream: 11.34 -> 11.0 ms).  Same results bit for bit.  At most 16
   streams can be marked at a time; unmark (on = 0) before destroying the stream.  No counterpart in the reference, which
   runs one stream. */
MCN_API int mcn_stream_beside(mcn_stream_t stream, int on);

/* Live per-kernel timing with HIP events on the stream the kernel is launched on.  After
   mcn_profile_begin("name"), every launch of the kernel family whose name contains "name" (e.g.
   "conv_pix_mfma", "conv_wgrad_mfma", "bnorm_sums", "bnorm_backward_apply", "pool_backward") is bracketed
   by a pair of events.  mcn_profile_end waits for the last one and reports the number of bracketed
   launches and the sum of their durations in milliseconds.  Not part of the reference interface (the
   reference relies on nvprof brackets, matlab/src/vl_cudatool.cu:126-131). */
MCN_API int mcn_profile_begin(const char* kernel_name);
MCN_API int mcn_profile_end(int* launches, double* total_ms);

/* Streaming yardstick (a measurement aid, not part of the reference interface): one launch of a plain kernel that
   reads `bytes` from src (MCN_YARDSTICK_READ; dst = one float that is never written in practice), writes them to
   dst (WRITE) or copies src to dst (COPY), with `width` bytes per access (4, 8, 16), `inFlight` accesses issued per
   lane before the first is used (1, 2, 4, 8), `blocks` workgroups of 256 threads (0: one step each) and flags
   (MCN_YARDSTICK_NONTEMPORAL: stores with the non-temporal hint; MCN_YARDSTICK_CHUNKED: every workgroup walks a
   contiguous run of its own instead of sharing the array slab by slab).  Timed with mcn_profile_begin("yardstick").
   The best of a sweep, with cold caches, is the measured ceiling the bandwidth-bound operators are reported
   against beside the nominal 8 TB/s; the copy of known size scales the HBM byte counters. */
enum { MCN_YARDSTICK_READ = 0, MCN_YARDSTICK_WRITE = 1, MCN_YARDSTICK_COPY = 2 };
enum { MCN_YARDSTICK_NONTEMPORAL = 1, MCN_YARDSTICK_CHUNKED = 2 };
MCN_API int mcn_hbm_yardstick(mcn_stream_t stream, void* dst, const void* src, size_t bytes, int mode, int width,
                              int inFlight, int blocks, int flags);

/* Matrix-pipe yardstick (no counterpart in the reference): one workgroup of sixteen wavefronts per CU, every wavefront a
   dependent chain of `iters` x 8 v_mfma_f32_32x32x2_f32 (isDouble: `iters` x 16 v_mfma_f64_16x16x4_f64) and nothing
   else; *flop receives the floating-point operations of the launch.  Timed with
   mcn_profile_begin("mfma_yardstick"): what it reaches is the measured ceiling the matrix-bound kernels are reported
   against beside the nominal peak (the chip does not hold its nominal clock under such a stream).  sink: one float
   of device memory, never written in practice. */
MCN_API int mcn_mfma_yardstick(mcn_stream_t stream, void* sink, int iters, int isDouble, double* flop);

/* ------------------------------------------------------------------------------------------------
 * convolution -- replaces ConvolutionForward/Backward<VLDT_GPU,T> (bits/nnconv.cu:71-157,163-317),
 * i.e. im2row_gpu + cublasSgemm per image, and the cuDNN variant (bits/nnconv_cudnn.cu:40-540).
 * ---------------------------------------------------------------------------------------------- */

MCN_API int mcn_conv_output_size(const mcn_conv_geom* g, int* outH, int* outW);

/* scratch bytes needed by one of the four products below (may be 0) */
MCN_API size_t mcn_conv_workspace_bytes(const mcn_conv_geom* g, int product);

/* y = outMult*y + inMult*conv(x,f) + b   (bits/nnconv.cu:71-157).  bias may be NULL.  When outMult is
   0 the previous contents of y are ignored (BLAS beta = 0 rule). */
MCN_API int mcn_conv_forward(mcn_stream_t stream, const mcn_conv_geom* g, float* y, float outMult,
                             const float* x, float inMult, const float* filters, const float* bias,
                             void* workspace, size_t workspaceBytes);

/* dzdx: H x W x C x N, fully overwritten  (bits/nnconv.cu:247-277: gemm 'n','t' + im2row::backward) */
MCN_API int mcn_conv_backward_data(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput,
                                   const float* filters, const float* derOutput, void* workspace,
                                   size_t workspaceBytes);

/* dzdx accumulated: derInput = derInputMult*derInput + dzdx (derInputMult = 0: same as mcn_conv_backward_data,
   previous contents ignored).  The reference has no such call: where a variable feeds several layers its
   derivatives are added by the network wrapper afterwards (matlab/+dagnn/Layer.m:130-132,
   "net.vars(v).der = net.vars(v).der + derInputs{i}"); this folds that addition into the convolution's output
   pass. */
MCN_API int mcn_conv_backward_data_acc(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput,
                                       float derInputMult, const float* filters, const float* derOutput,
                                       void* workspace, size_t workspaceBytes);

/* Filter banks packed ahead.  The matrix kernels read the filters re-laid ("packed": rows = reduction index in the
   order the kernel walks it, columns = output channels, padded to the tile).  mcn_conv_forward / mcn_conv_backward_data
   pack into their workspace on every call -- a launch of a few microseconds that a 53-layer network pays 80 times per
   step.  A caller whose filters stay put between calls (a network between two parameter updates, or for good when
   it only evaluates) can pack once into a buffer of its own and hand it to the *_packed calls.  No counterpart in
   the reference, whose GEMMs read the bank as stored (bits/nnconv.cu:126-134,256-264).
     mcn_conv_packed_bytes   size of that buffer for one product (MCN_CONV_FORWARD or MCN_CONV_BACKWARD_DATA) of one
                             geometry; 0 when the product reads no packed bank (direct kernels; 1x1 banks that
                             backward-data reads as stored).  The layout depends on the whole geometry, N included.
     mcn_conv_pack_filters   fills it (one launch per bank: one per filter group and stride class).
     mcn_conv_pack_plan / _layout / _batch   the same for many layers in one launch: _plan appends the jobs of one
                             product to a host array (filters and packed are the device addresses the jobs will
                             read and write), _layout numbers the workgroups of all jobs and returns their total,
                             and _batch, given a copy of the array in device memory, runs them all.
     mcn_conv_forward_packed, mcn_conv_backward_data_packed   as mcn_conv_forward / mcn_conv_backward_data_acc, reading
                             the banks from `packed` (NULL: pack on the fly as usual).  `filters` is still needed (banks
                             that are read as stored).  The packed buffer must have been filled from these filters
                             for this geometry and product: a stale buffer gives stale results. */
typedef struct { unsigned long long opaque[10]; } mcn_conv_pack_job;
MCN_API size_t mcn_conv_packed_bytes(const mcn_conv_geom* g, int product);
MCN_API int mcn_conv_pack_filters(mcn_stream_t stream, const mcn_conv_geom* g, int product, const float* filters,
                                  void* packed, size_t packedBytes);
MCN_API int mcn_conv_pack_plan(const mcn_conv_geom* g, int product, const float* filters, void* packed, size_t packedBytes,
                               mcn_conv_pack_job* jobs, int maxJobs, int* nJobs);
MCN_API unsigned mcn_conv_pack_layout(mcn_conv_pack_job* jobs, int nJobs);
MCN_API int mcn_conv_pack_batch(mcn_stream_t stream, const mcn_conv_pack_job* deviceJobs, int nJobs, unsigned totalBlocks);
MCN_API int mcn_conv_forward_packed(mcn_stream_t stream, const mcn_conv_geom* g, float* y, float outMult, const float* x,
                                    float inMult, const float* filters, const void* packed, size_t packedBytes,
                                    const float* bias, void* workspace, size_t workspaceBytes);
MCN_API int mcn_conv_backward_data_packed(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, float derInputMult,
                                          const float* filters, const void* packed, size_t packedBytes,
                                          const float* derOutput, void* workspace, size_t workspaceBytes);

/* Forward convolution that also sums its output per channel -- the first pass of a batch normalisation that
   follows it (bits/nnbnorm.cu:46-71 sums x and x^2 over the tensor the convolution has just written), taken from
   the accumulators while they are still in registers.  No counterpart in the reference, which runs the two layers
   one after the other.
     mcn_conv_forward_sums_groups   partial sums per channel the call below writes for this geometry; 0: this
                                    geometry has no such form (banks that do not fit in local memory, filter groups):
                                    use mcn_conv_forward and mcn_bnorm_forward
     mcn_conv_forward_sums          y = conv(x, filters) (no bias, y overwritten; `packed` as in mcn_conv_forward_packed,
                                    may be NULL) and sums[(k*groups + g)*2 + {0,1}] = partial sum of y and of y^2 over
                                    the pixels partial g covers, channel k, in double; K*groups*16 bytes.  The
                                    partials are deterministic (fixed by the launch shape); they are fp32 sums of at
                                    most a few hundred values each, widened to double.
   mcn_bnorm_forward_sums (below) takes them in place of its own summing pass. */
MCN_API int mcn_conv_forward_sums_groups(const mcn_conv_geom* g);
MCN_API int mcn_conv_forward_sums(mcn_stream_t stream, const mcn_conv_geom* g, float* y, const float* x, const float* filters,
                                  const void* packed, size_t packedBytes, double* sums, size_t sumsBytes, void* workspace,
                                  size_t workspaceBytes);

/* dzdx = conv backward-data (as mcn_conv_backward_data_packed with derInputMult = 0) + the derivative that reaches x
   along a second path, behind a ReLU: addend where its bit in maskBits is set (layout as mcn_bnorm_forward_sums_mask
   writes it, over a tensor of dzdx's shape), else addend*0.  In a residual block: the identity shortcut's share of the
   derivative, added in the epilogue of the first convolution's input gradient instead of being written out masked and
   read back.  Bit-identical to mcn_relu_backward into dzdx followed by mcn_conv_backward_data_packed with
   derInputMult = 1.  mcn_conv_backward_data_masked_add_supported: 1 when the geometry has this form (a filter bank that
   fits in local memory, whole 32-channel blocks, planes of a multiple of 32 elements), else 0 and the call fails.
   No counterpart in the reference. */
MCN_API int mcn_conv_backward_data_masked_add_supported(const mcn_conv_geom* g);
MCN_API int mcn_conv_backward_data_masked_add(mcn_stream_t stream, const mcn_conv_geom* g, float* derInput, const float* filters,
                                              const void* packed, size_t packedBytes, const float* derOutput,
                                              const float* addend, const unsigned* maskBits, void* workspace,
                                              size_t workspaceBytes);

/* dzdf: FH x FW x FC x K, fully overwritten  (bits/nnconv.cu:280-311: im2row::forward + gemm 't','n'
   accumulated over images) */
MCN_API int mcn_conv_backward_filter(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters,
                                     const float* x, const float* derOutput, void* workspace,
                                     size_t workspaceBytes);

/* Filter gradients whose final sum is deferred.  mcn_conv_backward_filter is two launches: the matrix kernel, which
   leaves one partial bank per reduction split in the workspace, and a sum over the splits of a few microseconds --
   which a network pays once per layer.  A caller that needs the gradients only at the end of its backward pass can
   keep each layer's partial banks in a buffer of its own and sum all layers in ONE launch.  No counterpart in the
   reference (its GEMM accumulates over images with beta = 1, bits/nnconv.cu:300-308).
     mcn_conv_backward_filter_partial_bytes   size of the buffer of partial banks for this geometry (0: the deferred
                                              form is not available; use mcn_conv_backward_filter)
     mcn_conv_backward_filter_plan            the jobs (one per filter group) that will sum `partials` into derFilters
     mcn_conv_backward_filter_partial         the matrix kernel alone; derFilters is written only by the later sum
                                              (or at once, when the geometry needs no sum at all: then no job exists)
     mcn_conv_reduce_layout / _batch          number the workgroups of many jobs; run them all, given the array in
                                              device memory.  Same bits as mcn_conv_backward_filter. */
typedef struct { unsigned long long opaque[6]; } mcn_conv_reduce_job;
MCN_API size_t mcn_conv_backward_filter_partial_bytes(const mcn_conv_geom* g);
MCN_API int mcn_conv_backward_filter_plan(const mcn_conv_geom* g, float* derFilters, void* partials, size_t partialBytes,
                                          mcn_conv_reduce_job* jobs, int maxJobs, int* nJobs);
MCN_API int mcn_conv_backward_filter_partial(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters, const float* x,
                                             const float* derOutput, void* partials, size_t partialBytes);
MCN_API unsigned mcn_conv_reduce_layout(mcn_conv_reduce_job* jobs, int nJobs);
MCN_API int mcn_conv_reduce_batch(mcn_stream_t stream, const mcn_conv_reduce_job* deviceJobs, int nJobs, unsigned totalBlocks);

/* dzdb: K values, fully overwritten  (bits/nnconv.cu:230-244: gemv with the all-ones vector) */
MCN_API int mcn_conv_backward_bias(mcn_stream_t stream, const mcn_conv_geom* g, float* derBias,
                                   const float* derOutput, void* workspace, size_t workspaceBytes);

/* dzdf and dzdb by one call: what vl::nn::Convolution::backward computes when both DERFILTERS and DERBIASES are asked
   for (bits/nnconv.cu:230-244,280-311).  For first layers (at most four input channels, a filter volume of at most 159
   elements, 32 or 64 filters) one pass over x and dzdy gives both; other layers run the two products above one after
   the other.  Workspace: the larger of mcn_conv_workspace_bytes for MCN_CONV_BACKWARD_FILTER and
   MCN_CONV_BACKWARD_BIAS.  Same results as the two separate calls to rounding (another summation order). */
MCN_API int mcn_conv_backward_filter_bias(mcn_stream_t stream, const mcn_conv_geom* g, float* derFilters, float* derBias,
                                          const float* x, const float* derOutput, void* workspace, size_t workspaceBytes);

/* ------------------------------------------------------------------------------------------------
 * subsampling with bias -- vl_nnconv with empty FILTERS (the identity filter bank, vl_nnconv.cu:316-321,432-441):
 * replaces Subsample::forwardWithBias / backwardWithBias (bits/nnsubsample.cu:31-216, nnsubsample_gpu.cu).
 * Output extent: (H + padTop + padBottom - 1)/strideY + 1, likewise for the width.
 * ---------------------------------------------------------------------------------------------- */

MCN_API int mcn_subsample_output_size(int H, int W, int strideY, int strideX, int padTop, int padBottom,
                                      int padLeft, int padRight, int* outH, int* outW);

/* y[oh,ow,c,n] = x[oh*strideY - padTop, ow*strideX - padLeft, c, n] (0 outside x) + bias[c]; bias may be NULL */
MCN_API int mcn_subsample_forward(mcn_stream_t stream, float* y, const float* x, const float* bias, int H, int W,
                                  int C, int N, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                                  int padRight);

/* dzdx (H x W x C x N, fully overwritten): dzdy placed back on the sampled positions, 0 elsewhere.  The bias
   derivative of this layer is mcn_conv_backward_bias on dzdy. */
MCN_API int mcn_subsample_backward(mcn_stream_t stream, float* derInput, const float* derOutput, int H, int W,
                                   int C, int N, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                                   int padRight);

/* y[h,w,c,n] += bias[c] in place -- the bias step of ConvolutionTranspose forward (bits/nnconv.cu:369-371,
   vl::nn::Bias::forward with both multipliers 1, bits/nnbias.cu) */
MCN_API int mcn_bias_add(mcn_stream_t stream, float* y, const float* bias, int H, int W, int C, int N);

/* ------------------------------------------------------------------------------------------------
 * batch normalisation -- replaces BatchNorm*<VLDT_GPU,T> (bits/nnbnorm_gpu.cu:818-1188).
 * `moments` is C x 2: C means followed by C sigmas, sigma = sqrt(var + epsilon) (bits/nnbnorm.cu:65-70).
 * ---------------------------------------------------------------------------------------------- */

MCN_API size_t mcn_bnorm_workspace_bytes(int H, int W, int C, int N);

/* givenMoments == 0: moments are computed from the batch and, if `moments` is non-NULL, written there
   (BatchNorm::forward, bits/nnbnorm.cu:201-256).  givenMoments != 0: `moments` is an input
   (forwardWithMoment, :170-199). */
MCN_API int mcn_bnorm_forward(mcn_stream_t stream, float* y, float* moments, const float* x,
                              const float* multipliers, const float* biases, int H, int W, int C, int N,
                              double epsilon, int givenMoments, void* workspace, size_t workspaceBytes);

/* Same as mcn_bnorm_forward with the element-wise layers that usually follow folded into the output pass:
   y = act(bnorm(x) [+ residual]), act = ReLU when relu != 0 (matlab/vl_nnrelu.m:43-48), residual added as
   matlab/+dagnn/Sum.m:11-17 would.  Every element takes the same roundings as with separate calls, so the
   result is bit-identical to mcn_bnorm_forward + mcn_add + mcn_relu_forward; two passes over the tensor are
   saved per folded layer.  No counterpart in the reference, which runs these layers one by one. */
MCN_API int mcn_bnorm_forward_fused(mcn_stream_t stream, float* y, float* moments, const float* x,
                                    const float* multipliers, const float* biases, const float* residual,
                                    int relu, int H, int W, int C, int N, double epsilon, int givenMoments,
                                    void* workspace, size_t workspaceBytes);

/* mcn_bnorm_forward_fused (moments from the batch) whose summing pass has been done already by the layer that
   produced x: `sums` holds sumGroups partial sums of x and x^2 per channel as mcn_conv_forward_sums writes them.  Only
   the output pass runs.  `moments` (may be NULL) receives the batch moments. */
MCN_API int mcn_bnorm_forward_sums(mcn_stream_t stream, float* y, float* moments, const float* x, const float* multipliers,
                                   const float* biases, const float* residual, int relu, int H, int W, int C, int N,
                                   double epsilon, const double* sums, int sumGroups);

/* The derivative of "batch normalisation, then ReLU" in one go: derOutput is dz/d(ReLU output), and it counts only
   where the layer's own output g*(x - mean)/sigma + b was positive, which is recomputed from x and the moments the
   forward pass stored (mcn_bnorm_forward* normalise with exactly those stored values, so the sign comes out the
   same bit for bit).  Otherwise as mcn_bnorm_backward with givenMoments != 0; results are bit-identical to
   mcn_relu_backward on the forward output followed by mcn_bnorm_backward, without writing and re-reading the
   masked derivative.  No counterpart in the reference, which runs these layers one by one
   (matlab/vl_nnrelu.m, bits/nnbnorm.cu:263-305). */
MCN_API int mcn_bnorm_backward_relu(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                                    const float* moments, const float* x, const float* multipliers,
                                    const float* biases, const float* derOutput, int H, int W, int C, int N,
                                    double epsilon, void* workspace, size_t workspaceBytes);

/* Batch-norm derivative (given moments) whose incoming derivative first passes the derivative of a ReLU that sits
   later in the network, behind other layers (in a residual block: behind the shortcut sum), so that the mask cannot
   be recomputed from x: maskedDerOutput = derOutput where maskSource > 0, else derOutput*0 (maskSource: that ReLU's
   output or input; as mcn_relu_backward), written out because the other consumers of that ReLU's derivative need it
   too, and summed in the same pass over the data.  Bit-identical to mcn_relu_backward followed by
   mcn_bnorm_backward with givenMoments != 0; one sweep of the tensor less.  No counterpart in the reference. */
MCN_API int mcn_bnorm_backward_masked(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                                      const float* moments, const float* x, const float* multipliers,
                                      const float* derOutput, const float* maskSource, float* maskedDerOutput,
                                      int H, int W, int C, int N, double epsilon, void* workspace,
                                      size_t workspaceBytes);

/* The same, with the later ReLU's mask as one bit per element instead of a tensor of floats -- a thirty-second of the
   bytes on each of the backward sweeps that need it, and no masked copy of the derivative written out.
     mcn_bnorm_mask_bits_supported  1 when tensors of this shape can carry such a mask (planes of a multiple of 32
                                    elements, large enough to be walked 16 bytes per lane), else 0
     mcn_bnorm_forward_sums_mask    mcn_bnorm_forward_sums with the ReLU on, which also writes maskBits: bit e % 32 of
                                    word e / 32 is set when element e of y (in memory order) is > 0; H*W*C*N/8 bytes
     mcn_bnorm_backward_bits        mcn_bnorm_backward_masked reading maskBits where that reads maskSource; nothing else
                                    is written (the other consumers of the masked derivative take derOutput and
                                    maskBits themselves: mcn_conv_backward_data_masked_add).  Bit-identical to it.
   No counterpart in the reference. */
MCN_API int mcn_bnorm_mask_bits_supported(int H, int W, int C, int N);
MCN_API int mcn_bnorm_forward_sums_mask(mcn_stream_t stream, float* y, unsigned* maskBits, float* moments, const float* x,
                                        const float* multipliers, const float* biases, const float* residual, int H, int W,
                                        int C, int N, double epsilon, const double* sums, int sumGroups);
MCN_API int mcn_bnorm_backward_bits(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                                    const float* moments, const float* x, const float* multipliers, const float* derOutput,
                                    const unsigned* maskBits, int H, int W, int C, int N, double epsilon, void* workspace,
                                    size_t workspaceBytes);

/* dzdx (H x W x C x N), dzdg (C), dzdb (C), all fully overwritten.  givenMoments == 0: BatchNorm::backward
   (bits/nnbnorm.cu:307-365), moments written if non-NULL.  givenMoments != 0: backwardWithMoment (:263-305). */
MCN_API int mcn_bnorm_backward(mcn_stream_t stream, float* derInput, float* derMultipliers,
                               float* derBiases, float* moments, const float* x,
                               const float* multipliers, const float* derOutput, int H, int W, int C,
                               int N, double epsilon, int givenMoments, void* workspace,
                               size_t workspaceBytes);

/* mcn_bnorm_backward for callers that cannot allocate device memory and have no workspace to hand over (code under
   HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
   arguments, meaning and bits as mcn_bnorm_backward without the workspace: the per-channel partial sums go to a device
   array built into the library (MCN_BNORM_STATIC_SCRATCH_BYTES per device, held until the process ends).  The call
   allocates and frees nothing; its first call on a device looks up that device's copy of the array (make that call
   outside graph capture).  Shapes whose partial sums do not fit (mcn_bnorm_workspace_bytes(H,W,C,N) >
   MCN_BNORM_STATIC_SCRATCH_BYTES) are rejected with MCN_UNSUPPORTED before anything is launched.  Every call on a
   device uses the same array: two calls that overlap on one device (different streams, different threads) race;
   calls on one stream are ordered and need nothing cleared between them. */
#define MCN_BNORM_STATIC_SCRATCH_BYTES (1u << 20)
MCN_API int mcn_bnorm_backward_static(mcn_stream_t stream, float* derInput, float* derMultipliers, float* derBiases,
                                      float* moments, const float* x, const float* multipliers, const float* derOutput,
                                      int H, int W, int C, int N, double epsilon, int givenMoments);

/* ------------------------------------------------------------------------------------------------
 * pooling -- replaces PoolingForward/Backward<VLDT_GPU,T> (bits/nnpooling_gpu.cu:270-415).
 * ---------------------------------------------------------------------------------------------- */

MCN_API int mcn_pool_output_size(const mcn_pool_geom* g, int* outH, int* outW);

MCN_API int mcn_pool_forward(mcn_stream_t stream, const mcn_pool_geom* g, float* y, const float* x);

/* accumulate != 0: derInput += pooling'(derOutput), the contract of vl::nn::Pooling::backward, whose
   caller zero-fills derInput first (vl_nnpool.cu:255-259).  accumulate == 0: derInput is write-only and
   receives exactly what the reference produces from a zero-filled buffer, so the separate fill pass
   can be dropped.  Either way the result is deterministic and, for max pooling, bit-identical to the
   reference CPU loop (first maximum in memory order wins, bits/nnpooling.cu:47-53,190-206). */
MCN_API int mcn_pool_backward(mcn_stream_t stream, const mcn_pool_geom* g, float* derInput,
                              const float* x, const float* derOutput, int accumulate);

/* ------------------------------------------------------------------------------------------------
 * element-wise companions used between the operators above
 * ---------------------------------------------------------------------------------------------- */

/* y = max(x, 0); dzdx = dzdy .* (x > 0)   (matlab/vl_nnrelu.m:43-48, leak = 0) */
MCN_API int mcn_relu_forward(mcn_stream_t stream, float* y, const float* x, size_t n);
MCN_API int mcn_relu_backward(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, size_t n);
/* the same with a leak: y = x .* (leak + (1 - leak)*(x > 0)), dzdx = dzdy .* (leak + (1 - leak)*(x > 0))
   (matlab/vl_nnrelu.m:49-55; leak = 0 takes the plain form above) */
MCN_API int mcn_relu_forward_leaky(mcn_stream_t stream, float* y, const float* x, size_t n, double leak);
MCN_API int mcn_relu_backward_leaky(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, size_t n,
                                    double leak);
/* y = a + b   (matlab/+dagnn/Sum.m:11-17; also the fan-out derivative sum of +dagnn/Layer.m:127-135) */
MCN_API int mcn_add(mcn_stream_t stream, float* y, const float* a, const float* b, size_t n);
/* y = alpha*a + beta*b, the momentum / weight update of SGD (matlab/src/vl_taccummex.cu:48-78: copy, BLAS scal, then
   BLAS axpy; examples/cnn_train_dag.m:316-378).  y may be a (the MEX's 'InPlace' mode).  Each element goes through
   the roundings of that pair: t = fl(alpha*a), y = fl(t + fl(beta*b)). */
MCN_API int mcn_taccum(mcn_stream_t stream, float* y, float alpha, const float* a, float beta, const float* b, size_t n);
/* SGD with momentum, the default solver of examples/cnn_train_dag.m:335-364, over all parameters of a network in one
   launch instead of three vl_taccum calls per parameter.  value / state / der are arenas of `chunks` chunks of
   MCN_SGD_CHUNK floats; each parameter occupies whole chunks (padded with zeros), chunk c belongs to parameter
   chunkParam[c] (device array), and rates[2p], rates[2p+1] (device array of doubles) are that parameter's learningRate
   and weightDecay multipliers (net.params(p).learningRate / .weightDecay).  Per element, with
   thisLR = (float)(learningRate*rates[2p]), thisDecay = (float)(weightDecay*rates[2p+1]) and the roundings of the
   reference's calls (each vl_taccum is t = fl(alpha*a), y = fl(t + fl(beta*b))):
     d     = vl_taccum(derScale, der, thisDecay, value)        derScale = 1/numWorkers (:344)
     state = vl_taccum(momentum, state, -1, d)                 (:350)
     value = vl_taccum(1, value, thisLR, nesterov ? fl(fl(momentum*state) - d) : state)   (:355-362)
   Parameters with thisLR = thisDecay = 0 are left alone (:342).  der is not modified. */
#define MCN_SGD_CHUNK 1024
MCN_API int mcn_sgd_momentum(mcn_stream_t stream, float* value, float* state, const float* der, size_t chunks,
                             const unsigned short* chunkParam, const double* rates, double learningRate,
                             double weightDecay, double momentum, double derScale, int nesterov);
/* y[i] = value   (bits/impl/copy_gpu.cu:17-33 fill) */
MCN_API int mcn_fill(mcn_stream_t stream, float* y, float value, size_t n);

/* ------------------------------------------------------------------------------------------------
 * losses -- matlab/vl_nnloss.m:136-317 (MATLAB code on gpuArrays in the reference; the last layers of
 * examples/imagenet/cnn_imagenet_init_resnet.m:128-139 are three of them: 'softmaxlog', 'classerror', 'topkerror').
 * x is H x W x C x N.  Categorical losses take one label (a class number 1..C as a float; 0 = skip this instance)
 * per image (nLabels == N) or per prediction vector (nLabels == H*W*N); attribute losses take one label (+1 / -1;
 * 0 = skip) per element of x.  instanceWeights (may be NULL) multiply the terms; their nWeights values are
 * broadcast over the labels by index (H*W values: one map for all images; 1: a scalar; as many as labels: one each).
 * normalise != 0 divides by N, as the reference does for 4-D inputs.
 * ---------------------------------------------------------------------------------------------- */
enum {
  MCN_LOSS_CLASSERROR = 0, MCN_LOSS_TOPKERROR = 1, MCN_LOSS_LOG = 2, MCN_LOSS_SOFTMAXLOG = 3, MCN_LOSS_MHINGE = 4,
  MCN_LOSS_MSHINGE = 5, MCN_LOSS_BINARYERROR = 6, MCN_LOSS_BINARYLOG = 7, MCN_LOSS_LOGISTIC = 8, MCN_LOSS_HINGE = 9
};
typedef struct mcn_loss_geom {
  int H, W, C, N;
  int loss;          /* MCN_LOSS_* */
  int topK;          /* 'topkerror' (reference default 5) */
  int normalise;     /* reference default: true */
  double threshold;  /* 'binaryerror' (reference default 0) */
} mcn_loss_geom;
MCN_API size_t mcn_loss_workspace_bytes(const mcn_loss_geom* g);
/* y[0] (device) = sum over the instances of weight * loss term  (vl_nnloss.m:229-271) */
MCN_API int mcn_loss_forward(mcn_stream_t stream, const mcn_loss_geom* g, float* y, const float* x, const float* labels,
                             size_t nLabels, const float* instanceWeights, size_t nWeights, void* workspace,
                             size_t workspaceBytes);
/* dzdx (shape of x, fully overwritten) for the scalar derOutput = dz/dy  (vl_nnloss.m:273-316) */
MCN_API int mcn_loss_backward(mcn_stream_t stream, const mcn_loss_geom* g, float* derInput, const float* x,
                              const float* labels, size_t nLabels, const float* instanceWeights, size_t nWeights,
                              double derOutput);

/* softmax over the channels (matlab/vl_nnsoftmax.m:20-28; the 'prob' layer a deployed network ends with):
   y = exp(x - max) / sum;  dzdx = y .* (dzdy - sum over the channels of dzdy .* y) */
MCN_API int mcn_softmax_forward(mcn_stream_t stream, float* y, const float* x, int H, int W, int C, int N);
MCN_API int mcn_softmax_backward(mcn_stream_t stream, float* derInput, const float* x, const float* derOutput, int H, int W,
                                 int C, int N);

/* ------------------------------------------------------------------------------------------------
 * double precision -- the operators' VLDT_Double instantiation (bits/impl/dispatcher.hpp:60-98 switches on the
 * tensors' data type; bits/nnconv.cu:444-469, bits/nnbnorm.cu:388-442, bits/nnpooling.cu:270-282 instantiate
 * every product for float and double).  Same arguments and meaning as the single-precision calls above; general
 * kernels (any geometry, one accumulator per output element), not tuned ones.  Pooling results have the bits of
 * the reference's sequential CPU loops.  The convolution calls need no workspace; the batch-normalisation calls
 * need 2*C doubles of workspace only when `moments` is NULL.
 * ---------------------------------------------------------------------------------------------- */
MCN_API int mcn_conv_forward_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* y, double outMult, const double* x,
                                 double inMult, const double* filters, const double* bias);
MCN_API int mcn_conv_backward_data_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derInput, const double* filters,
                                       const double* derOutput);
MCN_API int mcn_conv_backward_filter_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derFilters, const double* x,
                                         const double* derOutput);
MCN_API int mcn_conv_backward_bias_f64(mcn_stream_t stream, const mcn_conv_geom* g, double* derBias,
                                       const double* derOutput);
MCN_API int mcn_bnorm_forward_f64(mcn_stream_t stream, double* y, double* moments, const double* x,
                                  const double* multipliers, const double* biases, int H, int W, int C, int N,
                                  double epsilon, int givenMoments, void* workspace, size_t workspaceBytes);
MCN_API int mcn_bnorm_backward_f64(mcn_stream_t stream, double* derInput, double* derMultipliers, double* derBiases,
                                   double* moments, const double* x, const double* multipliers, const double* derOutput,
                                   int H, int W, int C, int N, double epsilon, int givenMoments, void* workspace,
                                   size_t workspaceBytes);
MCN_API int mcn_pool_forward_f64(mcn_stream_t stream, const mcn_pool_geom* g, double* y, const double* x);
MCN_API int mcn_pool_backward_f64(mcn_stream_t stream, const mcn_pool_geom* g, double* derInput, const double* x,
                                  const double* derOutput, int accumulate);
/* the companions in double: subsampling with bias (bits/nnsubsample.cu:31-216), the per-channel bias add of
   ConvolutionTranspose (bits/nnconv.cu:369-371), vl_taccum (matlab/src/vl_taccummex.cu:48-113) */
MCN_API int mcn_subsample_forward_f64(mcn_stream_t stream, double* y, const double* x, const double* bias, int H, int W,
                                      int C, int N, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                                      int padRight);
MCN_API int mcn_subsample_backward_f64(mcn_stream_t stream, double* derInput, const double* derOutput, int H, int W, int C,
                                       int N, int strideY, int strideX, int padTop, int padBottom, int padLeft,
                                       int padRight);
MCN_API int mcn_bias_add_f64(mcn_stream_t stream, double* y, const double* bias, int H, int W, int C, int N);
MCN_API int mcn_taccum_f64(mcn_stream_t stream, double* y, double alpha, const double* a, double beta, const double* b,
                           size_t n);

#ifdef __cplusplus
}
#endif
#endif /* MCN_HIP_H */
