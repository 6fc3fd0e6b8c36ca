/*
 * shadow_hip.h -- C ABI of the MI355X (gfx950) device layer for Shadow's tensor
 * hot path: Unary, Binary (N-d broadcast), Eltwise, Reduce, Activate, Scale and
 * the elementwise part of Blas.
 *
 * Conventions
 *   - every entry point returns int: 0 on success, a positive hipError_t value
 *     when the HIP runtime failed, a negative SHDW_E_* value when the arguments
 *     were rejected on the host before anything was enqueued.
 *     shdw_hip_error_string() turns either into text.
 *   - nothing throws, nothing synchronises unless its name says "sync" (the
 *     one exception, shdw_hip_asum, is documented at its declaration).
 *   - `stream` is a hipStream_t passed as void*; NULL means the null stream.
 *   - all tensors are dense row-major fp32 in device memory; element counts
 *     and indices are int32 like Shadow's Blob::count().
 *   - pointers are borrowed for the duration of the enqueued work.  Every
 *     purely elementwise entry point may be called in place (y == a).
 *   - arithmetic follows Shadow's CPU kernels exactly: separate multiply and
 *     add (never fused), std::max/std::min selection semantics, fp64
 *     accumulation in reductions.
 *
 * Citations "ref:" name the file and lines of junluan/shadow that the entry
 * point replaces on the GPU side.
 */
#ifndef SHADOW_HIP_H_
#define SHADOW_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes produced by this library itself (hipError_t are > 0) ---- */
#define SHDW_OK 0
#define SHDW_E_INVALID_ARGUMENT (-1) /* null pointer, negative count, bad enum */
#define SHDW_E_UNSUPPORTED (-2)      /* shape outside what the kernels accept  */
#define SHDW_E_WORKSPACE (-3)        /* workspace missing or too small         */
#define SHDW_E_STATIC_SCRATCH (-4)   /* needs more than the library's static scratch */

/* ---- operation enums; values are Shadow's ---- */
/* ref: shadow/operators/kernels/unary.hpp:9-25 */
enum {
  SHDW_UNARY_ABS = 0, SHDW_UNARY_SQUARE = 1, SHDW_UNARY_SQRT = 2, SHDW_UNARY_LOG = 3,
  SHDW_UNARY_EXP = 4, SHDW_UNARY_SIN = 5, SHDW_UNARY_COS = 6, SHDW_UNARY_TAN = 7,
  SHDW_UNARY_ASIN = 8, SHDW_UNARY_ACOS = 9, SHDW_UNARY_ATAN = 10, SHDW_UNARY_FLOOR = 11,
  SHDW_UNARY_CEIL = 12, SHDW_UNARY_NEG = 13, SHDW_UNARY_RECIPROCAL = 14
};
/* ref: shadow/operators/kernels/binary.hpp:23 */
enum {
  SHDW_BINARY_ADD = 0, SHDW_BINARY_SUB = 1, SHDW_BINARY_MUL = 2, SHDW_BINARY_DIV = 3,
  SHDW_BINARY_POW = 4, SHDW_BINARY_MAX = 5, SHDW_BINARY_MIN = 6
};
/* ref: shadow/operators/kernels/eltwise.hpp:9 */
enum { SHDW_ELTWISE_PROD = 0, SHDW_ELTWISE_SUM = 1, SHDW_ELTWISE_MAX = 2, SHDW_ELTWISE_MIN = 3 };
/* ref: shadow/operators/kernels/reduce.hpp:21-29 */
enum {
  SHDW_REDUCE_PROD = 0, SHDW_REDUCE_SUM = 1, SHDW_REDUCE_MAX = 2, SHDW_REDUCE_MIN = 3,
  SHDW_REDUCE_AVG = 4, SHDW_REDUCE_L1 = 5, SHDW_REDUCE_L2 = 6
};
/* ref: shadow/operators/kernels/activate.hpp:24-34 */
enum {
  SHDW_ACT_PRELU = 0, SHDW_ACT_RELU = 1, SHDW_ACT_LEAKY = 2, SHDW_ACT_SIGMOID = 3,
  SHDW_ACT_SOFTPLUS = 4, SHDW_ACT_TANH = 5, SHDW_ACT_RELU6 = 6, SHDW_ACT_HARDSWISH = 7,
  SHDW_ACT_GELU = 8
};

/* ======================= device, stream, allocator ======================= */

/* ref: shadow/core/context.cu:87-92 (check_device: cudaGetDeviceCount) */
int shdw_hip_device_count(int* count);
/* ref: shadow/core/context.cu:15,63 (cudaSetDevice in ctor and switch_device) */
int shdw_hip_set_device(int device_id);
/* ref: shadow/core/context.cu:93-101 (cudaGetDeviceProperties for the debug line).
 * Writes "name|gcnArch|CUs|clock_khz" into buf (truncated to buf_size). */
int shdw_hip_device_info(int device_id, char* buf, size_t buf_size);
/* ref: shadow/core/context.cu:17-21 (cudaStreamCreate) */
int shdw_hip_stream_create(void** stream);
/* ref: shadow/core/context.cu:39-43 (cudaStreamDestroy) */
int shdw_hip_stream_destroy(void* stream);
/* ref: shadow/core/context.cu:65-67 (cudaStreamSynchronize) */
int shdw_hip_stream_sync(void* stream);
/* ref: shadow/core/external.hpp:39-43 (CUDA_CHECK -> cudaGetErrorString) */
const char* shdw_hip_error_string(int rc);
/* ref: shadow/core/external.hpp:39-43 together with the cudaPeekAtLastError
 * after each launch (e.g. shadow/core/blas.cu:20): returns and clears the
 * runtime's sticky launch error. */
int shdw_hip_last_error(void);

/* ref: shadow/core/allocator.cu:11-18 (GPUAllocator::malloc -> cudaMalloc) */
int shdw_hip_malloc(void** ptr, size_t bytes);
/* ref: shadow/core/allocator.cu:47 (GPUAllocator::free -> cudaFree) */
int shdw_hip_free(void* ptr);
/* Free and total memory of the current device (hipMemGetInfo).  No counterpart in
 * the reference: it lets a caller, and the tests, see that an entry point which
 * promises not to allocate leaves the device's free memory as it was. */
int shdw_hip_mem_info(size_t* free_bytes, size_t* total_bytes);
/* ref: shadow/core/allocator.cu:29-36 (write: H2D; blocking when stream==NULL) */
int shdw_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream);
/* ref: shadow/core/allocator.cu:20-27 (read: D2H; blocking when stream==NULL) */
int shdw_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream);
/* ref: shadow/core/allocator.cu:38-45 (copy: D2D; blocking when stream==NULL) */
int shdw_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
/* Pinned host staging memory for the two calls above; Shadow reads back into a
 * pageable std::vector (shadow/core/blob.hpp:52-63), which makes its D2H
 * effectively blocking. */
int shdw_hip_host_malloc(void** ptr, size_t bytes);
int shdw_hip_host_free(void* ptr);

/* Events: Shadow only times on the host (Util::Timer, shadow/util/util.hpp:529-657);
 * the measurement harness needs device time for one stream. */
int shdw_hip_event_create(void** event);
int shdw_hip_event_destroy(void* event);
int shdw_hip_event_record(void* event, void* stream);
int shdw_hip_event_sync(void* event);
int shdw_hip_event_elapsed_ms(void* start, void* stop, float* ms);

/* Reads the n / 4 whole vectors of x, one per lane, and writes nothing, except `sentinel` to *sink (device memory) from a
 * lane whose four values add up to it.  With shdw_hip_copy and shdw_hip_set it
 * gives the harness the read, copy and write ceilings of a tensor size; the
 * reference has no counterpart. */
int shdw_hip_probe_read(int n, const float* x, float sentinel, float* sink, void* stream);

/* ============================ Blas, elementwise ========================== */

/* y[i] = val.  ref: shadow/core/blas.cpp:25-34, shadow/core/blas.cu:11-21 */
int shdw_hip_set(int n, float val, float* y, void* stream);
/* y[i] = f(a[i]), f chosen by SHDW_UNARY_*.
 * ref: shadow/core/blas.cpp:143-168 (loop branch), shadow/core/blas.cu:77-108,
 *      dispatch shadow/operators/kernels/unary.hpp:37-93 */
int shdw_hip_unary(int operation, int n, const float* a, float* y, void* stream);
/* y[i] = a[i] op b[i], SHDW_BINARY_*.
 * ref: shadow/core/blas.cpp:103-121, shadow/core/blas.cu:23-48 */
int shdw_hip_binary(int operation, int n, const float* a, const float* b, float* y,
                    void* stream);
/* y[i] = a[i] op alpha.
 * ref: shadow/core/blas.cpp:123-141, shadow/core/blas.cu:50-75 */
int shdw_hip_binary_scalar(int operation, int n, const float* a, float alpha, float* y,
                           void* stream);
/* x[i] *= alpha.  ref: shadow/core/blas.cpp:172-184, blas.cu:110-115 */
int shdw_hip_scal(int n, float alpha, float* x, void* stream);
/* y[i] = x[i].    ref: shadow/core/blas.cpp:186-200, blas.cu:117-122 */
int shdw_hip_copy(int n, const float* x, float* y, void* stream);
/* y[i] += alpha * x[i] (separate fp32 multiply and add).
 * ref: shadow/core/blas.cpp:202-217, blas.cu:124-130 */
int shdw_hip_axpy(int n, float alpha, const float* x, float* y, void* stream);
/* *result_host = (float) sum_i |x[i]| accumulated in fp64.  Like cublasSasum
 * with a host result pointer this call returns only after the value is on the
 * host (it synchronises `stream`).  `workspace` must hold 16 bytes more than
 * shdw_hip_reduce_workspace_bytes(1, {n}, 1, {0}) (the device-side result).
 * ref: shadow/core/blas.cpp:219-235, blas.cu:132-138 */
int shdw_hip_asum(int n, const float* x, float* result_host, void* workspace,
                  size_t workspace_bytes, void* stream);

/* ================================ Binary ================================= */

/* Numpy-style broadcast: a_shape/b_shape/out_shape are HOST arrays of num_axes
 * ints, already rank-aligned (each a/b dim equals the out dim or is 1).
 * y[out index] = a[...] op b[...] with a as the left operand.
 * The dims are collapsed on the host and travel as kernel arguments; there is
 * no device-side shape table.
 * ref: shadow/operators/kernels/binary.cpp:30-52, binary.cu:28-64,
 *      caller shadow/operators/kernels/binary.hpp:80-98 */
int shdw_hip_broadcast_binary(int operation, int num_axes, const int* a_shape,
                              const int* b_shape, const int* out_shape, const float* a,
                              const float* b, float* y, void* stream);

/* =============================== Activate ================================ */

/* y[i] = act(x[i]) for SHDW_ACT_RELU .. SHDW_ACT_GELU (type 0 is shdw_hip_prelu).
 * ref: shadow/operators/kernels/activate.cpp:9-39, activate.cu:7-45 */
int shdw_hip_activate(int type, float slope, int n, const float* x, float* y,
                      void* stream);
/* y[i] = x[i] > 0 ? x[i] : x[i] * slope[c], c = (i / dim) % channels, or c = 0
 * when channel_shared.  n = outer * channels * dim.
 * ref: shadow/operators/kernels/activate.cpp:41-53, activate.cu:47-69 */
int shdw_hip_prelu(int n, int channels, int dim, int channel_shared, const float* x,
                   const float* slope, float* y, void* stream);

/* ================================= Scale ================================= */

/* c = (i / inner_num) % scale_num;
 *   scale && bias : y = x * scale[c] + bias[c]   (multiply, then add)
 *   scale only    : y = x * scale[c]
 *   bias only     : y = x + bias[c]
 * followed by y = y > 0 ? y : 0 when relu != 0 (the Scale -> Activate(type 1)
 * pair in one launch; Shadow has no such fused op, parity target is the pair).
 * ref: shadow/operators/kernels/scale.cpp:7-39, scale.cu:7-67 */
int shdw_hip_scale_bias(int n, int scale_num, int inner_num, const float* x,
                        const float* scale, const float* bias, int relu, float* y,
                        void* stream);

/* ================================ Eltwise ================================ */

/* K >= 2 same-shape inputs, one pass.  xs is a HOST array of k device pointers,
 * coeff a HOST array of k floats (used by SUM only, may be NULL = all ones).
 *   PROD/MAX/MIN : acc = op(x0, x1); acc = op(acc, x_j) ...
 *   SUM          : acc = 0; acc = acc + coeff[j] * x_j ... (each step a separate
 *                  multiply and add, starting from +0 like Set + Saxpy)
 * When y aliases an input the result is what Shadow's pass-by-pass evaluation
 * gives: SUM overwrites y first, so an aliased input j reads as the running sum
 * (acc += coeff[j] * acc); for the other ops an aliased input j >= 2 reads as acc.
 * ref: shadow/operators/kernels/eltwise.hpp:18-71 */
int shdw_hip_eltwise(int operation, int k, const float* const* xs, const float* coeff,
                     int n, float* y, void* stream);
/* The same followed by Activate(relu) on the result, in the same pass: the
 * residual add and ReLU that close a block of a converted network whose
 * normalisation was folded into the convolution (the Native backend's fusion
 * pass calls this one).  Results are those of shdw_hip_eltwise followed by
 * shdw_hip_activate(relu) in place.
 * ref: shadow/operators/kernels/eltwise.hpp:18-71, activate.cpp:11-12 */
int shdw_hip_eltwise_relu(int operation, int k, const float* const* xs, const float* coeff,
                          int n, float* y, void* stream);

/* ================================= Reduce ================================ */

/* Bytes of device scratch shdw_hip_reduce needs for this shape/axes (0 when the
 * shape runs in a single stage).  in_shape and axes are HOST arrays.
 * Shadow sizes its temp buffer the same way before the launch:
 * ref: shadow/operators/kernels/reduce.hpp:72-76 (GrowTempBuffer) */
size_t shdw_hip_reduce_workspace_bytes(int num_axes, const int* in_shape, int num_reduce,
                                       const int* axes);
/* y[o] = reduce over the listed axes; one output per combination of the kept
 * axes, row-major.  Axes must be distinct and in [0, num_axes).  PROD, SUM,
 * AVG, L1, L2 accumulate in fp64 and round once; MAX/MIN return the first
 * element (in Shadow's list order) that attains the extremum and skip NaNs,
 * starting from lowest()/max().
 * ref: shadow/operators/kernels/reduce.cpp:9-76, reduce.cu:7-83,
 *      host planning shadow/operators/kernels/reduce.hpp:41-88 */
int shdw_hip_reduce(int operation, int num_axes, const int* in_shape, int num_reduce,
                    const int* axes, const float* x, float* y, void* workspace,
                    size_t workspace_bytes, void* stream);

/* shdw_hip_reduce for callers that cannot allocate device memory or pass a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments,
 * results and kernels as shdw_hip_reduce; the partial results of sliced shapes
 * go to a buffer inside the library's own device memory (1 MiB on every GPU the
 * library runs on, held until the process ends) instead of a workspace, and the
 * call allocates nothing.  A shape whose partials need more than
 * shdw_hip_reduce_static_max_workspace_bytes() is rejected with
 * SHDW_E_STATIC_SCRATCH and nothing is launched.  All calls on one GPU share the
 * buffer: calls that overlap in time on one GPU (different streams, different
 * threads) race; calls on one stream are ordered and safe.  The buffer's address
 * is looked up once per device, by shdw_hip_set_device or else by the first call
 * of this entry point on that device: a caller that captures a stream makes
 * either of the two before the capture begins. */
int shdw_hip_reduce_static(int operation, int num_axes, const int* in_shape, int num_reduce,
                           const int* axes, const float* x, float* y, void* stream);
size_t shdw_hip_reduce_static_max_workspace_bytes(void);

/* ============================ fused sequences ============================ */

/* Scale(blob form) -> Eltwise SUM with a residual -> Activate(relu) ->
 * Reduce AVG over the trailing `inner_num` elements, in one launch:
 *   c = row % scale_num;  s = x*scale[c] + bias[c];
 *   y = relu((0 + 1*s) + 1*residual);  mean[row] = (float)(sum_fp64(y) / inner_num)
 * rows = n / inner_num.  y may be NULL when only the pooled output is wanted.
 * Shadow runs these as four operators; parity target is that sequence:
 * ref: shadow/operators/kernels/scale.cpp:7-18, eltwise.hpp:37-44,
 *      activate.cpp:11-12, reduce.cpp:40-46 */
int shdw_hip_scale_residual_relu_rowmean(int n, int scale_num, int inner_num,
                                         const float* x, const float* scale,
                                         const float* bias, const float* residual,
                                         float* y, float* mean, void* stream);

/* The same sequence in the forms a converted network holds it in (the Native
 * backend's fusion pass calls this one): `scale` or `bias` may be NULL (the Scale
 * operator with has_scale or has_bias only: s = x*scale[c], or s = x + bias[c]);
 * residual_first != 0 when the residual is the Eltwise operator's first input,
 * y = relu((0 + 1*residual) + 1*s); `mean` may be NULL when no Reduce follows
 * (y is then required), `y` may be NULL when only the mean is wanted.
 * ref: shadow/operators/scale_op.cpp:25-33, eltwise_op.cpp:19-34,
 *      shadow/python/converter/shadow/optimizer.py:155-394 (where the reference fuses) */
int shdw_hip_scale_residual_relu(int n, int scale_num, int inner_num, const float* x,
                                 const float* scale, const float* bias, const float* residual,
                                 int residual_first, float* y, float* mean, void* stream);

/* The same sequence with a BatchNorm (global statistics) in front of the Scale,
 * how a Caffe-style model holds a bottleneck's last normalisation:
 *   c = row % channel;
 *   t = (x - stat_mean[c]*scale_factor) / sqrt(|stat_variance[c]*scale_factor| + eps);
 *   s = t*scale[c] + bias[c];  y and mean as above.
 * stat_mean, stat_variance, scale and bias hold `channel` values each (scale or
 * bias may be NULL, not both); every step is rounded as in the five operators.
 * ref: shadow/operators/kernels/batch_norm.cpp:11-24, batch_norm.cu:9-34 and
 *      the references of shdw_hip_scale_residual_relu */
int shdw_hip_batch_norm_scale_residual_relu(int n, int channel, int inner_num, const float* x,
                                            const float* stat_mean, const float* stat_variance,
                                            float scale_factor, float eps, const float* scale,
                                            const float* bias, const float* residual,
                                            int residual_first, float* y, float* mean,
                                            void* stream);

/* ==================== neighbouring operators of the path ==================== */

/* Axpy: out[r*inner_num + i] = y[..] + alpha[r] * x[..] for r < outer_num
 * (multiply, then add).  out may alias y; it must not alias x.
 * ref: shadow/operators/kernels/axpy.cpp:9-21 (memcpy + one BlasSaxpy per row),
 *      axpy.cu:7-26 */
int shdw_hip_axpy_rows(int outer_num, int inner_num, const float* alpha, const float* x,
                       const float* y, float* out, void* stream);

/* BatchNorm with global statistics: c = (i / inner_num) % channel;
 *   y = (x - mean[c]*scale_factor) / sqrt(|variance[c]*scale_factor| + eps)
 * with IEEE divide and square root.  y may alias x.
 * ref: shadow/operators/kernels/batch_norm.cpp:11-24, batch_norm.cu:9-34 */
int shdw_hip_batch_norm(int n, int channel, int inner_num, const float* x, const float* mean,
                        const float* variance, float scale_factor, float eps, float* y,
                        void* stream);

/* BatchNorm with global statistics followed by Scale over the same channel axis
 * (scale and bias hold `channel` values each; either may be null, not both) and,
 * with relu != 0, by Activate(relu), in one pass: per element
 *   t = (x - mean[c]*scale_factor) / sqrt(|variance[c]*scale_factor| + eps);
 *   t = t * scale[c];  t = t + bias[c];  y = relu ? (t > 0 ? t : 0) : t
 * -- the operators' own arithmetic, so the result is theirs bit for bit.  The pair
 * a Caffe-style model holds every normalisation in; Shadow has no such fused
 * operator (its converter folds the pair into the convolution where there is one,
 * python/converter/shadow/optimizer.py:181-252), the parity target is the sequence.
 * y may alias x.
 * ref: shadow/operators/kernels/batch_norm.cpp:11-24, scale.cpp:7-39,
 *      activate.cpp:12 */
int shdw_hip_batch_norm_scale(int n, int channel, int inner_num, const float* x, const float* mean,
                              const float* variance, float scale_factor, float eps,
                              const float* scale, const float* bias, int relu, float* y,
                              void* stream);

/* LRN across channels on a 4-D tensor [batch][channels][h][w]: per position a running
 * fp32 sum of the squares of `size` neighbouring channels (the entering square is
 * added, then the leaving one subtracted, channel after channel),
 *   scale = k + sum * (alpha / size);   y = x * powf(scale, -beta).
 * The reference's scale blob (a temp blob of the input's size) is not needed.
 * size must be odd; channels >= (size - 1) / 2 (with fewer the reference writes in
 * front of that blob); size > 63 returns SHDW_E_UNSUPPORTED.  y may alias x.
 * ref: shadow/operators/kernels/lrn.cpp:9-60, lrn.hpp:36-46, lrn.cu */
int shdw_hip_lrn(const int* in_shape, int size, float alpha, float beta, float k, const float* x,
                 float* y, void* stream);

/* GridSample: x [batch][channel][in_h][in_w], grid [batch][out_h][out_w][2] holding
 * (x, y) in [-1, 1], y [batch][channel][out_h][out_w]; the source coordinate is
 * (v + 1) / 2 * (extent - 1).  mode 0: the nearest cell (roundf), 1: the four cells
 * around it, weighted in the reference's order of operations.  padding_mode 0:
 * zeros outside the input, 1: coordinates clamped to the border.  Every index is
 * clamped before use, so no grid value reads outside x.  A float that fits no int
 * converts as in the reference's x86-64 build (INT_MIN); a NaN coordinate in mode 1,
 * with which the reference indexes outside its input, gives NaN.  y must not be x.
 * ref: shadow/operators/kernels/grid_sample.cpp:9-100, grid_sample.cu,
 *      shadow/operators/grid_sample_op.cpp:9-47 */
int shdw_hip_grid_sample(const int* in_shape, const int* out_shape, int mode, int padding_mode,
                         const float* x, const float* grid, float* y, void* stream);

/* Softmax over the middle extent of x viewed as [outer_num][dim][inner_num]:
 * running maximum, exp(x - max), fp32 running sum in index order, divide.  The
 * per-column scratch blob of the reference is not needed.  y may alias x.
 * ref: shadow/operators/kernels/softmax.cpp:10-42, softmax.hpp:29-41,
 *      softmax.cu:9-70 */
int shdw_hip_softmax(int outer_num, int dim, int inner_num, const float* x, float* y,
                     void* stream);

/* Normalize: y = x / max(norm_p(column), eps), the norm accumulated in fp64 in
 * index order; p == 1 and p == 2 have their own forms, any other p goes through
 * powf.  y may alias x.
 * ref: shadow/operators/kernels/normalize.cpp:10-43, normalize.hpp:29-38,
 *      normalize.cu:7-56 */
int shdw_hip_normalize(int outer_num, int dim, int inner_num, float p, float eps,
                       const float* x, float* y, void* stream);

/* SSDNormalize with its optional scale, one call for SSDNormalizeKernel::Run.
 *   across_spatial == 0: every position (b, s) is divided by
 *     (float) sqrt((double) sum_c x^2 + eps), the squares formed in fp32 and
 *     summed in fp64 in channel order (bit-exact);
 *   across_spatial != 0: every item b is multiplied by
 *     1 / sqrt((float) sum x^2 + eps), all fp32 after the fp64 sum; the sum is
 *     associated differently from the reference's loop (same contract as
 *     shdw_hip_asum).  Needs `workspace` of
 *     shdw_hip_ssd_normalize_workspace_bytes(...) bytes, 8-byte aligned; it is
 *     written and read on `stream`, nothing returns to the host.
 * scale: NULL, one value (channel_shared != 0: out *= scale[0]) or `channels`
 * values (out * scale[c]), applied to the normalised value as a second fp32
 * product.  It is read on the device: no synchronisation (the reference copies a
 * shared scale to the host first).  y may alias x.
 * ref: shadow/operators/kernels/ssd_normalize.hpp:36-83 (Square, Sasum, Mul,
 *      Sscal, Scale), ssd_normalize.cpp:7-29 (the oracle; ssd_normalize.cu:7-43 takes the
 *      square root in fp32 instead, sqrtf((float) sum + eps)) */
size_t shdw_hip_ssd_normalize_workspace_bytes(int batch, int channels, int spatial_dim,
                                              int across_spatial);
int shdw_hip_ssd_normalize(int batch, int channels, int spatial_dim, int across_spatial, float eps,
                           const float* x, const float* scale, int channel_shared, float* y,
                           void* workspace, void* stream);

/* Pooling over [N][C][H][W] (2d) or [N][C][D][H][W] (3d); shapes are HOST arrays
 * of 4 / 5 ints and out_shape is what the operator computed.  pool_type 0 = max
 * (start at lowest(), keep unless smaller), 1 = average: fp32 running sum in
 * window order divided by the window size clipped to input + pad.
 * ref: shadow/operators/kernels/pooling.cpp:7-42 (2d), :44-86 (3d), pooling.cu:7-126 */
int shdw_hip_pooling2d(const int* in_shape, int pool_type, int kernel_h, int kernel_w,
                       int stride_h, int stride_w, int pad_h, int pad_w, const int* out_shape,
                       const float* x, float* y, void* stream);
int shdw_hip_pooling3d(const int* in_shape, int pool_type, int kernel_d, int kernel_h,
                       int kernel_w, int stride_d, int stride_h, int stride_w, int pad_d,
                       int pad_h, int pad_w, const int* out_shape, const float* x, float* y,
                       void* stream);

/* GroupNorm / InstanceNorm / LayerNorm core: x viewed as [outer_num][inner_num];
 *   alpha = 1.f / inner_num
 *   mean = (float) sum_fp64(alpha * x)            var = (float) sum_fp64(alpha * (x-mean)^2)
 *   y = (x - mean) / sqrt(var + eps)              (products and differences in fp32)
 * then, when scale and bias are given (both or neither), with i the element
 * index in the whole tensor and c = (i / scale_inner) % scale_num:
 *   y = y * scale[c] + bias[c]                    (multiply, then add)
 * GroupNorm: outer = N*group, scale_num = C, scale_inner = H*W; InstanceNorm is
 * group = C; LayerNorm: inner = prod(normalized_shape) = scale_num, scale_inner = 1.
 * The fp64 sums are associated differently from the reference's serial loop
 * (contract 1e-5 relative, in practice identical).  y may alias x.
 * ref: shadow/operators/kernels/group_norm.hpp:41-86, layer_norm.hpp:22-69,
 *      group_norm.cpp:7-27, group_norm.cu:7-48, shadow/core/blas.cpp:238-247 */
int shdw_hip_group_norm(int outer_num, int inner_num, float eps, const float* x,
                        const float* scale, const float* bias, int scale_num, int scale_inner,
                        float* y, void* stream);

/* The same with scratch memory of the caller, for rows too long and too few to
 * give a workgroup each (GroupNorm with few groups at batch 1, LayerNorm over
 * C*H*W): with it such rows are cut into slices that three launches work on side
 * by side, fp64 partial sums going through the scratch.  `workspace` holds at
 * least shdw_hip_group_norm_workspace_bytes(outer_num, inner_num) bytes, 8-byte
 * aligned (0 bytes: the rows need none); NULL / fewer bytes: as
 * shdw_hip_group_norm, a workgroup per row.  The reference keeps mean, variance
 * and a squared copy of the input in temp blobs of the Workspace.
 * ref: shadow/operators/kernels/group_norm.hpp:49-72, layer_norm.hpp:30-55 */
size_t shdw_hip_group_norm_workspace_bytes(int outer_num, int inner_num);
int shdw_hip_group_norm_ws(int outer_num, int inner_num, float eps, const float* x,
                           const float* scale, const float* bias, int scale_num, int scale_inner,
                           float* y, void* workspace, size_t workspace_bytes, void* stream);

/* =============================== data movers =============================== */

/* dst[n*dst_pitch + dst_offset + p] = src[n*src_pitch + src_offset + p] for
 * n < outer, p < chunk (a chunk must lie inside its row on both sides).  One
 * call per input of Concat / per output of Slice / per input of Stack:
 *   Concat: outer = num_concats, chunk = src_pitch = in_axis*concat_size,
 *           dst_pitch = out_axis*concat_size, dst_offset = offset_axis*concat_size
 *   Slice : chunk = dst_pitch = out_axis*slice_size, src_pitch = in_axis*slice_size,
 *           src_offset = offset_axis*slice_size
 *   Stack : chunk = src_pitch = stack_size, dst_pitch = out_axis*stack_size,
 *           dst_offset = n*stack_size
 * ref: shadow/operators/kernels/concat.cpp:5-16, slice.cpp:5-16, stack.cpp:5-14,
 *      concat.cu:7-33, slice.cu:7-32, stack.cu:7-30 */
int shdw_hip_copy_chunks(int outer, int chunk, const float* src, int src_pitch, int src_offset,
                         float* dst, int dst_pitch, int dst_offset, void* stream);

/* x viewed as [outer_num][gather_dim][inner_num] -> y [outer_num][num_indexes][inner_num],
 * y[o][k][:] = x[o][indexes[k]][:].  indexes is a DEVICE array of int32; an entry
 * outside [0, gather_dim) gives zeros (the reference reads out of bounds).
 * ref: shadow/operators/kernels/gather.cpp:5-17, gather.cu:7-30 */
int shdw_hip_gather(int outer_num, int gather_dim, int inner_num, int num_indexes,
                    const int* indexes, const float* x, float* y, void* stream);

/* Channel c moves to (c % (channel/group)) * group + c / (channel/group).
 * ref: shadow/operators/kernels/shuffle_channel.cpp:5-21, shuffle_channel.cu:7-33 */
int shdw_hip_shuffle_channel(int batch, int channel, int spatial_dim, int group, const float* x,
                             float* y, void* stream);

/* Pads (positive) or crops (negative) the two trailing axes of [N][C][H][W];
 * paddings = top, bottom, left, right (HOST array of 4), new cells take `value`.
 * One pass; the reference fills the output with Blas::Set first.
 * ref: shadow/operators/kernels/pad.cpp:5-32, pad.hpp:24-40, pad.cu:7-43 */
int shdw_hip_pad(const int* in_shape, const int* paddings, float value, const float* x, float* y,
                 void* stream);

/* y = x with axes permuted: out axis j is in axis order[j] (HOST arrays, up to 8
 * axes).  The step tables the reference uploads per call are kernel arguments.
 * ref: shadow/operators/kernels/permute.cpp:5-20, permute.hpp:26-52, permute.cu:7-31 */
int shdw_hip_permute(int num_axes, const int* in_shape, const int* order, const float* x, float* y,
                     void* stream);

/* [N][C][H][W] -> [N][C*s*s][H/s][W/s]; type 0 = Darknet's index order, 1 = natural.
 * ref: shadow/operators/kernels/reorg.cpp:5-72, reorg.cu:7-75 */
int shdw_hip_reorg(const int* in_shape, int type, int stride, const float* x, float* y,
                   void* stream);

/* Resize of the two trailing axes; type 0 = nearest, 1 = bilinear (align_corners
 * as in the reference; half-pixel centres otherwise).  Coordinates and weights
 * are computed in fp32 in the reference's operation order, no fused operations.
 * SHDW_E_UNSUPPORTED for align_corners with a single output row or column.
 * ref: shadow/operators/kernels/resize.cpp:5-78, resize.cu:7-92 */
int shdw_hip_resize(const int* in_shape, const int* out_shape, int type, int align_corners,
                    const float* x, float* y, void* stream);

/* ============================ plan inspection ============================ */

/* Host-only: the collapsed form shdw_hip_broadcast_binary would launch with.
 * Writes up to 8 collapsed dims (outermost first) and both stride vectors;
 * returns the collapsed rank (0 = single element), or a negative SHDW_E_*. */
int shdw_hip_plan_broadcast(int num_axes, const int* a_shape, const int* b_shape,
                            const int* out_shape, int* dims, int* a_strides,
                            int* b_strides);
/* Host-only: how shdw_hip_reduce would run.  kind: 0 = rows (contiguous axis),
 * 1 = strided axis, 2 = generic N-d.  outer/reduce/inner are the collapsed
 * extents (generic: outer = outputs, reduce = window size, inner = 0);
 * splits = number of first-stage slices of the reduce extent. */
int shdw_hip_plan_reduce(int num_axes, const int* in_shape, int num_reduce,
                         const int* axes, int* kind, int* outer, int* reduce,
                         int* inner, int* splits);

/* Host-only: which family of kernels shdw_hip_softmax / shdw_hip_normalize /
 * shdw_hip_pooling2d would launch for a shape, decided by the same code that
 * launches (nothing is launched, no device is needed).  *path is one of
 * SHDW_PATH_* below, *variant the family's own parameter, *grid the number of
 * workgroups of the (first) launch.  Pointer alignment, which some families look
 * at for a choice of loads, is taken as 16 bytes.  Any of the three may be NULL.
 * They exist so that a change of a threshold shows up in a test: the operators
 * have no counterpart of them in the reference. */
enum {
  SHDW_PATH_NONE = 0,         /* nothing to do (an empty extent) */
  SHDW_PATH_ROWS = 1,         /* inner_num == 1, whole rows in a wave's LDS tile; variant = rows per wave */
  SHDW_PATH_ROWS_STREAM = 2,  /* inner_num == 1, rows streamed in chunks; variant = rows per wave */
  SHDW_PATH_SHORT_ROWS = 3,   /* slabs of up to 16 floats, four to a lane; variant = floats per slab */
  SHDW_PATH_QUADS = 4,        /* dim <= 4: four positions per lane in registers */
  SHDW_PATH_PACKED = 5,       /* several small slabs per workgroup in LDS; variant = slabs per workgroup */
  SHDW_PATH_LONG_SLAB = 6,    /* one slab per workgroup, streamed in chunks */
  SHDW_PATH_SLAB = 7,         /* one slab per workgroup, whole in LDS */
  SHDW_PATH_COLUMNS_REG = 8,  /* a column per lane in registers; variant = registers per column */
  SHDW_PATH_TILE = 9,         /* 2^variant positions x dim channels per workgroup in LDS */
  SHDW_PATH_TALL = 10,        /* 2^variant positions per workgroup, channels in chunks */
  SHDW_PATH_COLUMNS = 11,     /* a column per lane, two passes over memory */
  /* pooling */
  SHDW_PATH_POOL_PLANE_REDUCE = 20, /* global max: Reduce's row kernels */
  SHDW_PATH_POOL_PLANE = 21,        /* global pooling, planes in LDS */
  SHDW_PATH_POOL_PLANE_STREAM = 22, /* global average of long planes, streamed */
  SHDW_PATH_POOL_SMALL_PLANES = 23, /* whole planes in LDS; variant = 100 * separable + window unrolled for (0: loops) */
  SHDW_PATH_POOL_BAND = 24,         /* bands of input rows in LDS; variant = 100 * registers per lane + window unrolled for */
  SHDW_PATH_POOL_WINDOW = 25,       /* a lane per output, windows from memory */
  SHDW_PATH_POOL_HALVE = 26,        /* 3x3 / 2x2 at stride 2, output rows half as long as input rows of 4 m columns: no staging; variant = window side */
  SHDW_PATH_POOL_SAME = 27          /* 3x3 at stride 1 with pad 1 on rows of 4 m columns: no staging */
};
int shdw_hip_softmax_plan(int outer_num, int dim, int inner_num, int* path, int* variant,
                          unsigned* grid);
int shdw_hip_normalize_plan(int outer_num, int dim, int inner_num, float p, int* path,
                            int* variant, unsigned* grid);
int shdw_hip_pooling2d_plan(const int* in_shape, int pool_type, int kernel_h, int kernel_w,
                            int stride_h, int stride_w, int pad_h, int pad_w,
                            const int* out_shape, int* path, int* variant, unsigned* grid);

#ifdef __cplusplus
}
#endif

#endif /* SHADOW_HIP_H_ */
