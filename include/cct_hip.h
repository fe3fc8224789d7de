/*
 * cct_hip.h -- C ABI of the MI355X (gfx950) device driver for CaffeConTroll's lowering-based
 * convolution training path.
 *
 * Every entry point is what a `HIPDriver : DeviceDriver` placed next to the reference's CPUDriver
 * binds for one DeviceDriver member; the member it stands for is cited on each declaration
 * (paths relative to the CaffeConTroll tree).  Pointers named dst/src/A/B/C/x/y are DEVICE
 * pointers unless the comment says otherwise; argument structs are HOST structs passed by
 * pointer and copied by value into kernel arguments.  Tensors are dense fp32 in the
 * reference's Layout_CRDB (index = c + r*C + d*R*C + b*R*C*D, src/LogicalCube_impl.hxx:216-220).
 *
 * Error convention: the reference's drivers return void and assert(false) on error
 * (src/sched/DeviceDriver.h:48-51).  Here every function returns 0 on success or a non-zero
 * code (a hipError_t value, or CCT_HIP_EINVAL for rejected arguments); the C++ HIPDriver
 * wrapper turns non-zero into message + abort to keep the reference behaviour.
 * cct_hip_last_error() describes the most recent failure on the calling thread.
 *
 * Streams: all work is enqueued on one stream per process (the null stream until
 * cct_hip_set_stream is called).  Calls are asynchronous with respect to the host unless
 * stated; cct_hip_device_sync() waits for the stream.
 */
#ifndef CCT_HIP_H
#define CCT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CCT_HIP_EINVAL 100001

/* CBLAS enum values as used by the reference's cblas.h consumers. */
enum { CCT_ROW_MAJOR = 101, CCT_COL_MAJOR = 102, CCT_NO_TRANS = 111, CCT_TRANS = 112 };

/* struct PMapHelper, src/sched/DeviceHeader.h:25-35 -- identical field order. */
typedef struct cct_pmap_helper {
  size_t dR, dC, dD, dB; /* dst RCDB */
  size_t sR, sC, sD, sB; /* src RCDB */
  size_t dBR, dBC;       /* dst block */
  size_t sBR, sBC;       /* src block */
  size_t kR, kC, kD, kB; /* kernel RCDB */
  size_t stride;
  size_t padding;
} cct_pmap_helper;

/* struct _inverse_lower_cube_arg_helper, src/kernels/lowering.h:22-32 -- identical field order. */
typedef struct cct_inverse_lower_cube_args {
  size_t data_output_width;
  size_t data_output_height;
  size_t kernel_size;
  size_t stride;
  size_t padding;
  size_t iR, iC, iD, iB;
} cct_inverse_lower_cube_args;

/* struct _pool_forward_arg_helper / _pool_backward_arg_helper, src/kernels/pool.h:7-29
 * (the two reference structs have the same fields in the same order). max_index: device. */
typedef struct cct_pool_args {
  int stride;
  int kernel_size;
  int iR, iC, oR, oC, D, B;
  int *max_index;
} cct_pool_args;

/* struct _lrn_forward_arg_helper, src/kernels/lrn.h:7-15. denoms: device. */
typedef struct cct_lrn_forward_args {
  int iR, iC, iD, iB;
  int norm_window;
  int local_size;
  char *denoms;
} cct_lrn_forward_args;

/* struct _lrn_forward_normalize_arg_helper, src/kernels/lrn.h:17-21. */
typedef struct cct_lrn_forward_normalize_args {
  float alpha_over_size;
  float beta;
  char *denoms;
} cct_lrn_forward_normalize_args;

/* struct _lrn_backward_arg_helper, src/kernels/lrn.h:23-35. Pointers: device. */
typedef struct cct_lrn_backward_args {
  int oR, oC, oD, oB;
  float alpha_over_size;
  float beta;
  int norm_window;
  int local_size;
  char *denoms;
  char *input_data;
  char *output_data;
} cct_lrn_backward_args;

/* ---- process / device state --------------------------------------------------------- */
/* DeviceDriver::set_device_id + init_thread (src/sched/DeviceDriver.h:269-272): selects the
 * device for the calling thread and creates the library state on first use. */
int cct_hip_init(int device_id);
/* Use an existing hipStream_t (passed as void*) for all later work; NULL = null stream.  The
 * library works on ONE stream at a time: its split-K workspace and reduction counters are shared
 * by all calls, so work must not be spread over several streams by switching between them while
 * earlier calls are still running (synchronise before switching). */
int cct_hip_set_stream(void *hip_stream);
/* Tuning knobs, for experiments and for tests that pin a kernel instance.  Names: "direct_tile"
 * (<map blocks><pixel blocks> of the direct convolution tile, 161 / 162 = its 16-row variant with 128 / 256
 * pixels, 0 = automatic), "direct_waves",
 * "direct_tb", "direct_nospec", "direct_splits" (step ranges of the direct weight-gradient launch, 0 = automatic),
 * "direct_alds" (shape-specialised weight-gradient kernels: 1 = output-gradient rows staged in LDS, 2 = fetched by
 * their lanes, 0 = automatic), "direct_wgrad_rows" (stride-1 weight gradient: 1 = the image-pair kernels wherever they
 * apply, 2 = the one-image-per-step kernel always, 0 = automatic), "strided_wgrad" (tile of the strided weight-gradient kernel: pieces of an output row
 * x 1000 + column blocks x 100 + column groups x 10 + row blocks, 0 = automatic), "pool_plane", "gemm_nt", "gemm_tile" (-1 = automatic), "gemm_nodma" (1 = GEMM
 * operand tiles always staged through registers), "conv1x1_per_image" (1 x 1 layers, forward and data gradient: 1 = one
 * product per image, 2 = one product over the pixels of all images, 0 = automatic).  The
 * environment variables CCT_HIP_<NAME IN CAPITALS> give the initial values; they are read once,
 * when the library initialises, never on a launch path.  No counterpart in the reference. */
int cct_hip_set_tuning(const char *name, int value);
/* DeviceDriver::device_sync, src/sched/DeviceDriver.h:267. */
int cct_hip_device_sync(void);
const char *cct_hip_last_error(void);
/* The kernel instance the library chose for the most recent lowering, lifting, GEMM or direct
 * convolution call: kernel name with its template arguments as a kernel trace prints them, then
 * launch-time choices (e.g. "gemm_kernel<Tile<256,128,16,2,2>,true,false> splits=26").  For
 * harnesses that label measurements with what actually ran.  Kept per host thread: the text is
 * that of the calling thread's own last launch and stays valid until that thread's next one.  No
 * counterpart in the reference. */
const char *cct_hip_last_kernel(void);
/* Number of compute units of the selected device (0 before init). */
int cct_hip_compute_units(void);

/* ---- memory: DeviceDriver::malloc/free/memcpy/memset, src/sched/DeviceDriver.h:83-86 ---- */
int cct_hip_malloc(void **dev_ptr, size_t size_in_byte);
int cct_hip_free(void *dev_ptr);
/* kind: 0 host->device, 1 device->host, 2 device->device. Synchronous for kinds 0 and 1. */
int cct_hip_memcpy(void *dst, const void *src, size_t size_in_byte, int kind);
int cct_hip_memset(void *dev_ptr, int value, size_t size_in_byte);

/* ---- overlapped host <-> device staging ---------------------------------------------------- */
/* For a bridge whose layers live in host memory (ParallelizedBridge with share_pointer_with_prev_bridge /
 * share_pointer_with_next_bridge false, src/bridges/ParallelizedBridge_impl.hxx:595-621, 686-705, where
 * the reference issues blocking DeviceDriver::memcpy calls around the sub-bridge): a pipe is two side
 * streams, one per direction of the link, ordered against the library's compute stream by events, so that
 * the batch can move in pieces -- piece i+1 uploading and piece i-1 downloading while piece i computes.
 *   begin     uploads enqueued from here on start only after the kernels enqueued so far;
 *   upload    asynchronous host -> device copy on the upload stream; *ticket names it;
 *   wait_upload  kernels enqueued from here on start only after that upload has landed;
 *   download  asynchronous device -> host copy on the download stream, after the kernels enqueued so far;
 *   finish    the host waits for both side streams and the compute stream (tickets end here).
 * The copies overlap with kernels (and with each other) only from / to page-locked host memory
 * (hipHostMalloc, a pinned torch tensor); from pageable memory they are correct but serialise. */
typedef struct cct_hip_pipe cct_hip_pipe;
int cct_hip_pipe_create(cct_hip_pipe **pipe);
int cct_hip_pipe_destroy(cct_hip_pipe *pipe);
int cct_hip_pipe_begin(cct_hip_pipe *pipe);
int cct_hip_pipe_upload(cct_hip_pipe *pipe, void *dst_device, const void *src_host, size_t bytes, int *ticket);
int cct_hip_pipe_wait_upload(cct_hip_pipe *pipe, int ticket);
int cct_hip_pipe_download(cct_hip_pipe *pipe, void *dst_host, const void *src_device, size_t bytes);
int cct_hip_pipe_finish(cct_hip_pipe *pipe);

/* ---- lowering / lifting / remap ------------------------------------------------------ */
/* DeviceDriver::lower_cube<_fpmap_id,_fmap_lower> (src/sched/DeviceDriver.h:108-112; CPU
 * semantics src/sched/DeviceDriver_CPU.cpp:124-301).  src [sB][sD][sR][sC] ->
 * dst [sB*m*m][kR*kR*sD], whole batch in one launch, zero padding written explicitly. */
int cct_hip_lower_cube(float *dst, const float *src, const cct_pmap_helper *args);
/* DeviceDriver::inverse_lower_cube (src/sched/DeviceDriver.h:119-122; CPU semantics
 * src/sched/DeviceDriver_CPU.cpp:306-346).  src [iD*k*k][iB][oh*ow] -> dst [iB][iD][iR][iC].
 * Gather formulation: dst is overwritten (no prior zero fill needed) with the same per-pixel
 * summation order (kr ascending, kc ascending) as the reference's scatter loop. */
int cct_hip_inverse_lower_cube(float *dst, const float *src,
                               const cct_inverse_lower_cube_args *args);
/* inverse_lower_cube and backward_bias in ONE launch: the lift blocks gather dst from src while
 * extra blocks reduce out_grad [batch][depth][fmap] into bias_grad [depth] with wavefront
 * reductions.  Replaces the pair Connector::inverse_lower_cube
 * (src/Connector_impl_Lowering_type1.hxx:130-183) + bias gradient
 * (src/bridges/ConvolutionBridge_impl.hxx:575-599). */
int cct_hip_inverse_lower_cube_bias_backward(float *dst, const float *src,
                                             const cct_inverse_lower_cube_args *args,
                                             float *bias_grad, const float *out_grad,
                                             int fmap_size, int depth, int batch_size);
/* DeviceDriver::pmap2d_read_coalesce<_fpmap_id,_fmap_remap> (src/sched/DeviceDriver.h:100-104,
 * src/kernels/lowering.hxx:241-258): slice j of src (sR*sC floats, j < sD*sB) goes to slice
 * (j / sB) + (j % sB) * sD of dst.  dst and src must not overlap. */
int cct_hip_remap(float *dst, const float *src, const cct_pmap_helper *args);
/* The backward remap of a convolution's output gradient ([image][map] slices -> [map][image]
 * slices, src/bridges/ConvolutionBridge_impl.hxx:601-605) together with the bias gradient
 * (ConvolutionBridge_impl.hxx:575-599) in one pass over the tensor: source slice j belongs to map
 * j % sB, and bias_grad[o] (sB entries) = sum of every element of map o's slices.  Used when the
 * layer needs no input gradient (first layer), so no lifting kernel is there to carry the sum. */
int cct_hip_remap_bias_backward(float *dst, const float *src, const cct_pmap_helper *args, float *bias_grad);

/* Depth-slice copy between a contiguous cube part [B][d_count][rc] and channels
 * [d_off, d_off + d_count) of whole [B][d_total][rc]; gather != 0: whole -> part, else part -> whole.
 * Stands for the host loops of the reference's Split / Concat bridges used for grouped layers
 * (src/DeepNet.h:1700-1757, 1924-2028). */
int cct_hip_copy_depth_slice(float *part, float *whole, int B, int d_total, int d_off, int d_count,
                             size_t rc, int gather);

/* ---- BLAS-shaped ----------------------------------------------------------------------- */
/* DeviceDriver::sgemm (src/sched/DeviceDriver.h:206-208), cblas_sgemm contract. fp32 MFMA. */
int cct_hip_sgemm(int order, int TA, int TB, int M, int N, int K, float alpha, const float *A,
                  int lda, const float *B, int ldb, float beta, float *C, int ldc);
/* DeviceDriver::sgemm_new (src/sched/DeviceDriver.h:211-213): row-major,
 * lda = (TA==N ? K : M), ldb = (TB==N ? N : K), ldc = N. */
int cct_hip_sgemm_new(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                      const float *B, float beta, float *C);
/* cct_hip_sgemm_new followed by the bias over a 1 x 1 feature map, in one pass: the non-CPU branch of
 * FullyConnectedBridge::forward (src/bridges/FullyConnectedBridge_impl.hxx:224-228 -- sgemm_new, then
 * forward_bias).  C[m][n] = alpha * op(A) op(B) + beta * C[m][n] + col_bias[n] (col_bias may be NULL);
 * relu != 0 also applies the ReLU of a following in-place ReLUBridge (max(x, 0),
 * src/kernels/relu.hxx:10-25) before the store.  The sums are those of the two separate calls, in
 * the same order: identical results. */
/* sgemm_new, and beside it colsum[c] = sum over r of colsum_src[r][c] (rows x cols, dense row-major; rows ascending
 * within four quarters that are added in order: the same bits as cct_hip_backward_bias_fc).  The two
 * results are independent; the sums ride in spare workgroups of the product's reduction launch when it has one.
 * For FullyConnectedBridge::backward, which computes the bias gradient and the data gradient from the same
 * output gradient (src/bridges/FullyConnectedBridge_impl.hxx:268-308). */
int cct_hip_sgemm_new_colsum(int TA, int TB, int M, int N, int K, float alpha, const float *A, const float *B,
                             float beta, float *C, float *colsum, const float *colsum_src, int rows, int cols);
int cct_hip_sgemm_new_bias(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                           const float *B, float beta, float *C, const float *col_bias, int relu);
/* Forward-convolution GEMM with the output permutation and bias of
 * ConvolutionBridge::forward (src/bridges/ConvolutionBridge_impl.hxx:328-364) folded into the
 * epilogue: out[b][o][fmap] = model[o x K] * lowered[b*fmap x K]^T + bias[o] (bias may be NULL).
 * relu != 0 also applies the ReLU of a following in-place ReLUBridge (max(x, 0),
 * src/kernels/relu.hxx:10-25) before the store. */
int cct_hip_sgemm_conv_forward(int o, int batch, int fmap, int K, const float *model,
                               const float *lowered, const float *bias, float *out, int relu);
/* ---- inner-product layers with few outputs -------------------------------------------------- */
/* FullyConnectedBridge::forward / ::backward (src/bridges/FullyConnectedBridge_impl.hxx:169-234,
 * 255-326) for layers of at most 32 outputs at batches of at most 1024 (LeNet's 500 -> 10 classifier):
 * the sgemm_new + forward_bias of the forward pass as one launch, and the backward_bias_fc + two
 * sgemm_new of the backward pass as one launch, in plain fp32 multiply-adds (a 64 x 64 matrix-core
 * tile would be nearly all padding; the layer's time is launch latency).  x [batch][in], w [out][in],
 * y / dy [batch][out], all dense.
 * forward: y = x w^T + bias (bias may be NULL); relu != 0 clamps at zero (a following in-place ReLU).
 * backward: dw = dy^T x; db = column sums of dy (db may be NULL); dx = dy w unless dx is NULL, stored
 * as 0 wherever relu_data (same shape as dx: the layer's input, output of an in-place ReLU before the
 * layer) is not positive, if relu_data is given.  Fixed summation orders: run-to-run identical. */
int cct_hip_fc_small_supported(int batch, int in_features, int out_features);
int cct_hip_fc_small_forward(float *y, const float *x, const float *w, const float *bias, int batch,
                             int in_features, int out_features, int relu);
int cct_hip_fc_small_backward(float *dx, float *dw, float *db, const float *dy, const float *x, const float *w,
                              int batch, int in_features, int out_features, const float *relu_data);
/* ---- convolutions with a very short contraction and few maps --------------------------------- */
/* ConvolutionBridge::forward / ::backward (src/bridges/ConvolutionBridge_impl.hxx:294-373, 551-628) for stride-1
 * layers with one or three input channels, k = 3 or 5 and at most 32 output maps (LeNet's first layer): lowering,
 * GEMM, remap and bias of the forward pass as ONE launch that reads the model cube [o][d][k][k] as it is, and the
 * weight and bias gradient as one launch plus the fixed-order sum of its per-image-group partial sums, in plain
 * fp32 multiply-adds (k*k*d of 25 leaves a matrix-core tile mostly padding).  in [batch][d][n][n], out / dout
 * [batch][o][m][m], all dense; bias / db may be NULL; relu != 0 clamps the output at zero.  Results agree with
 * the other paths to fp32 rounding; run-to-run identical.  No data gradient (a first layer needs none; the
 * other kernels provide it otherwise). */
int cct_hip_conv_small_supported(int batch, int d, int n, int k, int stride, int pad, int o);
int cct_hip_conv_small_forward(float *out, const float *in, const float *w, const float *bias, int batch, int d, int n,
                               int k, int pad, int o, int relu);
int cct_hip_conv_small_backward_weights(float *dw, float *db, const float *dout, const float *in, int batch, int d,
                                        int n, int k, int pad, int o);
/* ---- 1 x 1 convolution without lowering --------------------------------------------------- */
/* A 1 x 1 filter at stride 1 without padding makes lower_cube a permuting copy: image i of the input
 * [batch][depth][plane] (plane = n*n) is already the depth x plane operand of its product.  These three replace
 * lower_cube + GEMM + remap_output + bias of ConvolutionBridge::forward (src/bridges/ConvolutionBridge_impl.hxx:294-373)
 * and remap + the two GEMMs + inverse_lower_cube + bias gradient of ::backward (:551-628) with products on the
 * tensors as they lie: forward and data gradient one product whose columns run over the pixels of all images (one
 * product per image, all in one launch, for planes above 2048 pixels or below 4), the weight gradient one product
 * summed over the images in a fixed order.  model [num_outputs][depth]; bias / bias_grad may
 * be NULL; relu != 0 clamps the output at zero.  Results agree with the lowering path to fp32 rounding.
 * cct_hip_conv1x1_supported: 1 for k == 1, stride == 1, padding == 0 (else 0: the lowering path takes the layer). */
int cct_hip_conv1x1_supported(int batch, int depth, int n, int k, int stride, int padding, int num_outputs);
int cct_hip_conv1x1_forward(float *output, const float *input, const float *model, const float *bias, int batch,
                            int depth, int plane, int num_outputs, int relu);
int cct_hip_conv1x1_backward_data(float *input_grad, const float *output_grad, const float *model, int batch,
                                  int depth, int plane, int num_outputs);
int cct_hip_conv1x1_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                     const float *input, int batch, int depth, int plane, int num_outputs);
/* ---- stride-1 convolution without the lowered matrix ------------------------------------ */
/* Fused replacements for chains of ConvolutionBridge's lowering pipeline when stride == 1 and
 * k is 3, 5 or 7.  Forward and data gradient take an image whose padded rows exceed 64 floats in column bands;
 * the weight gradient has image-pair kernels for padded rows of up to 32 floats and otherwise takes one image
 * per step and long output rows in up to 64 pieces (what bounds the width: a few thousand columns, fewer for a
 * layer with under 32 maps).  Results agree with the
 * lowering path to fp32 rounding (the sums run in another order), not bit for bit.
 * cct_hip_conv_direct_supported: 1 if both directions cover the geometry, else 0. */
int cct_hip_conv_direct_supported(int batch, int depth, int n, int k, int stride, int padding,
                                  int num_outputs);
/* Re-lays the model [o][d][k][k] into per-channel slabs: for_data_gradient == 0 gives
 * [d][o][k*k] (forward), != 0 gives [o][d][k*k] with every filter reversed.  Both slab dimensions
 * are padded with zeros (channels to a multiple of 4, maps to whole kernel tiles) so that the
 * convolution kernels read them without bounds tests: `slabs` must hold
 * cct_hip_conv_direct_slab_floats() floats and be 16-byte aligned. */
size_t cct_hip_conv_direct_slab_floats(int num_outputs, int depth, int k, int for_data_gradient);
int cct_hip_conv_direct_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                              int for_data_gradient);
/* The three kernels below take the distance in floats between consecutive images of the input
 * tensor and of the output tensor (input_image_stride, output_image_stride; 0 = dense, i.e.
 * d*n*n and o*m*m).  A larger stride addresses a channel slice of a wider tensor in place, which
 * is how a grouped convolution runs without gathering its slices
 * (DeepNet's Split/Concat grouping, src/DeepNet.h:1700-1757).
 *
 * lower_cube + forward GEMM + remap_output + bias of ConvolutionBridge::forward
 * (src/bridges/ConvolutionBridge_impl.hxx:316-364) in one kernel:
 * output[b][o][m][m] from input[b][d][n][n], forward slabs, bias[o] (may be NULL); relu != 0
 * folds a following in-place ReLU into the store. */
int cct_hip_conv_direct_forward(float *output, const float *input, const float *slabs,
                                const float *bias, int batch, int depth, int n, int k, int padding,
                                int num_outputs, size_t input_image_stride, size_t output_image_stride,
                                int relu);
/* Gradient remap + data-gradient GEMM + inverse_lower_cube of ConvolutionBridge::backward
 * (src/bridges/ConvolutionBridge_impl.hxx:601-616) in one kernel: input_grad[b][d][n][n] from
 * output_grad[b][o][m][m] (read in place, not permuted) and data-gradient slabs. */
int cct_hip_conv_direct_backward_data(float *input_grad, const float *output_grad, const float *slabs,
                                      int batch, int depth, int n, int k, int padding, int num_outputs,
                                      size_t input_image_stride, size_t output_image_stride);
/* The same followed by the backward of an in-place ReLU whose output is this layer's input
 * (src/bridges/ReLUBridge_impl.hxx:62-100, the next bridge DeepNet::run_backward_pass visits):
 * input_grad is stored as 0 wherever relu_data (the layer's input tensor, same shape and image
 * stride as input_grad) is not positive. */
int cct_hip_conv_direct_backward_data_relu(float *input_grad, const float *output_grad, const float *slabs,
                                           int batch, int depth, int n, int k, int padding, int num_outputs,
                                           size_t input_image_stride, size_t output_image_stride,
                                           const float *relu_data);
/* Weight-gradient GEMM of ConvolutionBridge::backward (src/bridges/ConvolutionBridge_impl.hxx:
 * 619-621) without the lowered matrix or the gradient remap: model_grad[o][d][k][k] (overwritten,
 * beta = 0) from output_grad[b][o][m][m] and input[b][d][n][n].  If bias_grad is not NULL the same
 * launch also produces the bias gradient bias_grad[o] = sum of output_grad over batch and pixels
 * (:575-599), in a fixed summation order. */
int cct_hip_conv_direct_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                         const float *input, int batch, int depth, int n, int k, int padding,
                                         int num_outputs, size_t input_image_stride, size_t output_image_stride);
/* The same five calls for a grouped convolution (`group` of cnn.proto's ConvolutionParameter; the
 * reference builds such a layer as towers between a Split and a Concat, src/DeepNet.h:1700-1757),
 * all groups in ONE launch: `depth` and `num_outputs` are the layer's totals, both divisible by
 * `groups`; group q convolves channels [q*depth/groups, (q+1)*depth/groups) of the input with
 * filters [q*num_outputs/groups, ...) of the model [num_outputs][depth/groups][k][k] (the blob
 * layout Caffe gives a grouped layer) into the same range of output maps.  The slab buffer holds
 * the groups' slabs one after another (cct_hip_conv_direct_slab_floats_grouped() floats in all);
 * model_grad / bias_grad have the model's / bias's layout.  Image strides as above, for the whole
 * tensors (0 = dense).  relu_data may be NULL (no ReLU mask).  With groups == 1 these ARE the
 * calls above.  Per element the sums run in the same order as in one call per group on channel
 * slices, so results are identical whenever both pick the same kernel instance and step ranges. */
int cct_hip_conv_direct_supported_grouped(int batch, int depth, int n, int k, int stride, int padding,
                                          int num_outputs, int groups);
size_t cct_hip_conv_direct_slab_floats_grouped(int num_outputs, int depth, int k, int for_data_gradient,
                                               int groups);
int cct_hip_conv_direct_slabs_grouped(float *slabs, const float *model, int num_outputs, int depth, int k,
                                      int for_data_gradient, int groups);
int cct_hip_conv_direct_forward_grouped(float *output, const float *input, const float *slabs,
                                        const float *bias, int batch, int depth, int n, int k, int padding,
                                        int num_outputs, size_t input_image_stride, size_t output_image_stride,
                                        int relu, int groups);
int cct_hip_conv_direct_backward_data_grouped(float *input_grad, const float *output_grad, const float *slabs,
                                              int batch, int depth, int n, int k, int padding, int num_outputs,
                                              size_t input_image_stride, size_t output_image_stride,
                                              const float *relu_data, int groups);
int cct_hip_conv_direct_backward_weights_grouped(float *model_grad, float *bias_grad, const float *output_grad,
                                                 const float *input, int batch, int depth, int n, int k,
                                                 int padding, int num_outputs, size_t input_image_stride,
                                                 size_t output_image_stride, int groups);
/* ---- strided convolution without the lowered matrix ---------------------------------------- */
/* The same replacement of ConvolutionBridge's lowering pipeline for strided layers: stride 4 with an
 * 11 x 11 kernel (AlexNet / CaffeNet conv1, benchmark configuration 3; the reference's "large" golden
 * scenario, tests/test_parallelized_convolution_large_CPU.cpp:71-80) and stride 2 with 7 x 7,
 * 5 x 5 or 3 x 3 kernels.  cct_hip_conv_strided_supported: 1 if the forward and the weight-gradient
 * kernel both cover the geometry (the layer can then run without the lowered matrix), else 0. */
int cct_hip_conv_strided_supported(int batch, int depth, int n, int k, int stride, int padding,
                                   int num_outputs);
/* Re-lays the model [o][d][k][k] for cct_hip_conv_strided_forward, zero padded: for a layer with
 * padding as [d][k rounded up to even][o padded to whole tiles][k+1 (+1)], for a layer without as
 * [d][pairs of tap rows][o padded to whole tiles][2k (+1)] (the two forward kernels read their
 * weights in different orders, so `padding` must be the layer's own); `slabs` holds
 * cct_hip_conv_strided_slab_floats() floats (0 if the kernel size / stride pair is not covered)
 * and is 16-byte aligned. */
size_t cct_hip_conv_strided_slab_floats(int num_outputs, int depth, int k, int stride, int padding);
int cct_hip_conv_strided_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                               int stride, int padding);
/* lower_cube + forward GEMM + remap_output + bias of ConvolutionBridge::forward
 * (src/bridges/ConvolutionBridge_impl.hxx:316-364) in one kernel: output[b][o][m][m],
 * m = (n + 2*padding - k) / stride + 1, from input[b][d][n][n], the slabs and bias[o] (may be NULL);
 * relu != 0 folds a following in-place ReLU into the store. */
int cct_hip_conv_strided_forward(float *output, const float *input, const float *slabs, const float *bias,
                                 int batch, int depth, int n, int k, int stride, int padding,
                                 int num_outputs, int relu);
/* Output-gradient remap + weight-gradient GEMM (+ bias gradient) of ConvolutionBridge::backward
 * (src/bridges/ConvolutionBridge_impl.hxx:575-604, 619-621) for a strided layer in one kernel plus a
 * fixed-order reduction of partial sums, reading the layer's input instead of the lowered matrix of
 * the forward pass: model_grad[o][d][k][k], bias_grad[o] (may be NULL) from output_grad[b][o][m][m]
 * and input[b][d][n][n]. */
int cct_hip_conv_strided_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                          const float *input, int batch, int depth, int n, int k,
                                          int stride, int padding, int num_outputs);
/* Output-gradient remap + data-gradient GEMM + inverse_lower_cube of ConvolutionBridge::backward
 * (src/bridges/ConvolutionBridge_impl.hxx:604-616) for a strided layer in one kernel: every
 * (row phase, column phase) sub-image of the input gradient is a stride-1 convolution of the output
 * gradient with ceil(k/stride)^2 of the filter's taps.  Covered: depth * stride^2 of at most 80 in an odd
 * number of 16-row blocks (3 x 16 for AlexNet / CaffeNet conv1), ceil(k/stride) <= 5, output gradient
 * rows of at most 64 - 2 (ceil(k/stride) - 1) floats.  The slabs (cct_hip_conv_strided_backward_data_slab_floats()
 * floats, 16-byte aligned) are rebuilt from the model [o][d][k][k] whenever it changes. */
int cct_hip_conv_strided_backward_data_supported(int batch, int depth, int n, int k, int stride, int padding,
                                                 int num_outputs);
size_t cct_hip_conv_strided_backward_data_slab_floats(int num_outputs, int depth, int k, int stride);
int cct_hip_conv_strided_backward_data_slabs(float *slabs, const float *model, int num_outputs, int depth,
                                             int k, int stride);
int cct_hip_conv_strided_backward_data(float *input_grad, const float *output_grad, const float *slabs,
                                       int batch, int depth, int n, int k, int stride, int padding,
                                       int num_outputs);
/* DeviceDriver::sgemv (src/sched/DeviceDriver.h:214-215): row-major M x N, lda = N. */
int cct_hip_sgemv(int TA, int M, int N, float alpha, const float *A, const float *x, float beta,
                  float *y);
/* DeviceDriver::math_saxpy / math_saxpby (src/sched/DeviceDriver.h:197,204): y = a*x (+ b*y). */
int cct_hip_math_saxpy(size_t n, float alpha, const float *x, float *y);
int cct_hip_math_saxpby(size_t n, float alpha, const float *x, float beta, float *y);
/* DeviceDriver::L1_update (src/sched/DeviceDriver.h:114-117). */
int cct_hip_L1_update(int n, float *gradient, float lambda, const float *model);
/* SGDGradientUpdater::update (src/algorithms/GradientUpdater.h:154-193) in one kernel:
 * g += lambda*w (or lambda*sign(w) when l1), h = stepsize*g + momentum*h, w -= h. */
int cct_hip_sgd_update(size_t n, float *model, float *gradient, float *history, float stepsize,
                       float momentum, float lambda, int l1);
/* The same update for several tensors in one launch: the updates DeepNet::run_backward_pass
 * (src/DeepNet.h:2012-2028) triggers layer by layer, collected and applied after the last layer's
 * backward (no layer reads another layer's weights in between, so the result is the same).  Meant
 * for the many small tensors (biases, small filters) whose separate launches cost more than their
 * arithmetic; every element sees exactly the arithmetic of cct_hip_sgd_update. */
typedef struct {
  size_t n;
  float *model, *gradient, *history;
  float stepsize, momentum, lambda;
  int l1;
} cct_sgd_job;
int cct_hip_sgd_update_batch(const cct_sgd_job *jobs, int count);
/* DeviceDriver::sconstant_initialize (src/sched/DeviceDriver.h:258-260). */
int cct_hip_sconstant_initialize(float *arr, size_t n, float value);
/* DeviceDriver::sinitialize_xavier / sbernoulli_initialize / sgaussian_initialize
 * (src/sched/DeviceDriver.h:242-256; CPUDriver src/sched/DeviceDriver_CPU.cpp:661-699): n floats
 * at the device pointer arr.  Drawn on the host the way CPUDriver draws them -- std::mt19937 seeded
 * with random_seed (std::random_device if -1), then one draw per element in index order from
 * uniform_real_distribution<float>(-s, s) with s = sqrt(3 / (n / n_batch)),
 * bernoulli_distribution(p), normal_distribution<float>(mean, std_dev) -- and copied to the device
 * (synchronous).  The cct_filler_draw_* forms write the same values to a HOST array and touch no
 * device. */
int cct_hip_fill_xavier(float *arr, size_t n, size_t n_batch, int random_seed);
int cct_hip_fill_bernoulli(float *arr, size_t n, float p, int random_seed);
int cct_hip_fill_gaussian(float *arr, size_t n, float mean, float std_dev, int random_seed);
int cct_filler_draw_xavier(float *host, size_t n, size_t n_batch, int random_seed);
int cct_filler_draw_bernoulli(float *host, size_t n, float p, int random_seed);
int cct_filler_draw_gaussian(float *host, size_t n, float mean, float std_dev, int random_seed);
/* DeviceDriver::rand_uint_initialize (src/sched/DeviceDriver.h:250-252) after init_rng(seed):
 * counter-based generator, word i of call c depends only on (seed, c, i). */
int cct_hip_init_rng(int random_seed);
int cct_hip_rand_uint_initialize(unsigned int *buf, int n);

/* ---- convolution / FC bias --------------------------------------------------------------- */
/* DeviceDriver::forward_bias (src/sched/DeviceDriver.h:124-127): out[b][d][fmap] += bias[d]. */
int cct_hip_forward_bias(const float *bias, float *out, int fmap_size, int depth, int batch_size);
/* DeviceDriver::backward_bias (src/sched/DeviceDriver.h:129-133): bias_grad[d] = sum_b sum_fmap. */
int cct_hip_backward_bias(float *bias_grad, const float *out_grad, int fmap_size, int depth,
                          int batch_size);
/* cct_hip_backward_bias for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arithmetic and summation order as cct_hip_backward_bias, but the partial sums and arrival
 * counters of the split reduction live in an array built into the library (80 KB per GPU, held
 * until the process ends) instead of the library's grow-only workspace: the call allocates and
 * frees nothing.  Limits: depth <= 4096 and depth x (batch split) <= 16384, else CCT_HIP_EINVAL.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
 * host threads) race. */
int cct_hip_backward_bias_noalloc(float *bias_grad, const float *out_grad, int fmap_size, int depth,
                                  int batch_size);
/* DeviceDriver::backward_bias_fc (src/sched/DeviceDriver.h:135-138): bias[d] = sum_b out[b][d]. */
int cct_hip_backward_bias_fc(float *bias_grad, const float *out_grad, int D, int B);

/* ---- elementwise / pooling / loss (the closed set of parallel_map UDF pairs the reference
 *      instantiates, src/sched/DeviceDriver_CPU.cpp:725-784, as named kernels) ------------- */
/* parallel_map<_f_src_to_dst_relu_forward,_f_relu_forward>, src/kernels/relu.hxx:10-28. */
int cct_hip_relu_forward(float *out, const float *in, size_t n);
/* parallel_map<_f_src_to_dst_relu_backward,_f_relu_backward>, src/kernels/relu.hxx:30-45. */
int cct_hip_relu_backward(float *in_grad, const float *out_grad, const float *in_data, size_t n);
/* DeviceDriver::maxpool_forward/backward, src/sched/DeviceDriver.h:149-156. dst is overwritten
 * (no -FLT_MAX pre-fill needed); backward overwrites in_grad (no zero fill needed). */
int cct_hip_maxpool_forward(float *out, const float *in, const cct_pool_args *args);
int cct_hip_maxpool_backward(float *in_grad, const float *out_grad, const cct_pool_args *args);
/* MaxPoolingBridge::backward followed by the backward of an in-place ReLU on the pooled tensor
 * (src/bridges/MaxPoolingBridge_impl.hxx:114-151 then src/bridges/ReLUBridge_impl.hxx:62-100, the
 * order DeepNet::run_backward_pass visits them): in_grad = pooling gradient where relu_data > 0,
 * else 0; relu_data is the pooled tensor (the ReLU's output), same shape as in_grad. */
int cct_hip_maxpool_backward_relu(float *in_grad, const float *out_grad, const cct_pool_args *args,
                                  const float *relu_data);
/* The same result from the pooling layer's OUTPUT tensor `pooled` (same shape as out_grad) instead
 * of its input: a gradient lands only on a window's arg-max, whose activation IS the window's
 * maximum, so switching off every window whose maximum is not positive gives the same sums, bit
 * for bit, and reads a tensor a quarter the size.  `pooled` must still hold the values
 * cct_hip_maxpool_forward wrote (a following in-place ReLU leaves their signs; in-place dropout
 * does not: use cct_hip_maxpool_backward_relu then). */
int cct_hip_maxpool_backward_relu_pooled(float *in_grad, const float *out_grad, const cct_pool_args *args,
                                         const float *pooled);
/* DeviceDriver::lrn_forward/lrn_backward, src/sched/DeviceDriver.h:140-147. */
int cct_hip_lrn_forward(float *out, const float *in, const cct_lrn_forward_args *args,
                        const cct_lrn_forward_normalize_args *args2);
int cct_hip_lrn_backward(float *in_grad, const float *out_grad, const cct_lrn_backward_args *args);
/* parallel_map<_f_src_to_dst_dropout_forward,_f_dropout_forward_train>,
 * src/kernels/dropout.hxx:20-32: out = in * (mask > threshold) * scale (in place allowed). */
int cct_hip_dropout_forward_train(float *out, const float *in, const unsigned int *mask,
                                  float scale, unsigned int threshold, size_t n);
/* parallel_map<_f_src_to_dst_softmax_forward,_f_softmax_forward>, src/kernels/softmax.hxx:19-60.
 * labels: device floats, one per image. loss_sum: device float, overwritten with the batch sum.
 * A label outside [0, len_per_image) is never used as an index: that image's loss (and so the
 * sum) becomes NaN, and the backward pass subtracts no 1 for it. */
int cct_hip_softmax_loss_forward(float *prob, const float *in, const float *labels,
                                 float *loss_sum, int len_per_image, int batch);
/* The forward pass above and the backward pass below in the same launch, for a training iteration that
 * will ask for the gradient anyway (SoftmaxLossBridge::forward then ::backward,
 * src/bridges/SoftmaxLossBridge_impl.hxx:36-84, 90-143): prob and loss_sum as cct_hip_softmax_loss_forward
 * writes them, in_grad as cct_hip_softmax_loss_backward would compute it from that prob.  Batches of a few
 * thousand scores in all (LeNet: 64 x 10) take one single-workgroup launch for everything. */
int cct_hip_softmax_loss_forward_backward(float *prob, float *in_grad, const float *in, const float *labels,
                                          float *loss_sum, int len_per_image, int batch, int spatial);
/* parallel_map<_f_src_to_dst_softmax_backward,_f_softmax_backward>, src/kernels/softmax.hxx:62-81:
 * in_grad = (prob - onehot(label)) / batch / spatial. */
int cct_hip_softmax_loss_backward(float *in_grad, const float *prob, const float *labels,
                                  int len_per_image, int batch, int spatial);

/* ---- timing on the library's stream (used by the harness; hipEvent based) ---------------- */
int cct_hip_timer_create(void **timer);
int cct_hip_timer_destroy(void *timer);
int cct_hip_timer_start(void *timer);
int cct_hip_timer_stop(void *timer);
/* Waits for the stop event; milliseconds between start and stop. */
int cct_hip_timer_elapsed_ms(void *timer, float *ms);

#ifdef __cplusplus
}
#endif
#endif /* CCT_HIP_H */
