// HIPDriver: the MI355X counterpart of the reference's CPUDriver / GPUDriver
// (src/sched/DeviceDriver.h:56-274, src/sched/DeviceDriver_CPU.h:24-111).  Same member names
// and argument meaning; every member forwards to the C ABI in include/cct_hip.h.
//
// Error behaviour follows src/sched/DeviceDriver.h:48-51: members return void; on error the
// message is printed and the process aborts (the reference asserts) -- unless the calling thread
// is inside an ErrorsAsExceptions scope (Fail.h), as the C entry points over the bridges are: then
// the member throws HostError with the same message.
//
// The reference selects kernels with C function pointers as template arguments
// (parallel_map<idx,func>).  The closed set of pairs it instantiates
// (src/sched/DeviceDriver_CPU.cpp:725-784) is provided here as named members instead, one per
// pair, so no device-side function pointers are needed.
#pragma once
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <random>
#include <string>
#include <vector>

#include "../../../include/cct_hip.h"
#include "Fail.h"
#include "DeviceMemoryPointer.h"

namespace cct {

typedef cct_pmap_helper PMapHelper;
typedef cct_inverse_lower_cube_args _inverse_lower_cube_arg_helper;
typedef cct_pool_args _pool_forward_arg_helper;
typedef cct_pool_args _pool_backward_arg_helper;
typedef cct_lrn_forward_args _lrn_forward_arg_helper;
typedef cct_lrn_forward_normalize_args _lrn_forward_normalize_arg_helper;
typedef cct_lrn_backward_args _lrn_backward_arg_helper;

enum CBLAS_ORDER { CblasRowMajor = CCT_ROW_MAJOR, CblasColMajor = CCT_COL_MAJOR };
enum CBLAS_TRANSPOSE { CblasNoTrans = CCT_NO_TRANS, CblasTrans = CCT_TRANS };

class HIPDriver {
 public:
  explicit HIPDriver(int device_id = 0) { ok(cct_hip_init(device_id), "init"); }

  // ---- pointers / memory (DeviceDriver.h:76-86) ----
  void *choose_ptr(void *host, void *device) { (void)host; return device; }
  DeviceMemoryPointer get_device_pointer(void *ptr, size_t size_in_byte) {
    return DeviceMemoryPointer_Local_GPURAM(ptr, size_in_byte);
  }
  void malloc(DeviceMemoryPointer *dst) { ok(cct_hip_malloc(&dst->ptr, dst->size_in_byte), "malloc"); }
  void free(DeviceMemoryPointer *dst) { ok(cct_hip_free(dst->ptr), "free"); dst->ptr = nullptr; }
  // direction is taken from the two pointer types, as GPUDriver::memcpy does
  void memcpy(DeviceMemoryPointer *dst, DeviceMemoryPointer *src) {
    const bool dd = dst->type == DEVICEMEMORY_LOCAL_GPURAM, sd = src->type == DEVICEMEMORY_LOCAL_GPURAM;
    if (!dd && !sd) { host_fail("HIPDriver::memcpy: host to host copy"); }
    const int kind = (dd && sd) ? 2 : dd ? 0 : 1;
    ok(cct_hip_memcpy(dst->ptr, src->ptr, dst->size_in_byte, kind), "memcpy");
  }
  void memset(DeviceMemoryPointer *dst, const char value) {
    ok(cct_hip_memset(dst->ptr, value, dst->size_in_byte), "memset");
  }
  // ---- overlapped staging of host-resident layers (no counterpart in DeviceDriver.h) ----
  cct_hip_pipe *pipe_create() {
    cct_hip_pipe *p = nullptr;
    ok(cct_hip_pipe_create(&p), "pipe_create");
    return p;
  }
  void pipe_destroy(cct_hip_pipe *p) { ok(cct_hip_pipe_destroy(p), "pipe_destroy"); }
  void pipe_begin(cct_hip_pipe *p) { ok(cct_hip_pipe_begin(p), "pipe_begin"); }
  int pipe_upload(cct_hip_pipe *p, void *dst_device, const void *src_host, size_t bytes) {
    int ticket = -1;
    ok(cct_hip_pipe_upload(p, dst_device, src_host, bytes, &ticket), "pipe_upload");
    return ticket;
  }
  void pipe_wait_upload(cct_hip_pipe *p, int ticket) { ok(cct_hip_pipe_wait_upload(p, ticket), "pipe_wait_upload"); }
  void pipe_download(cct_hip_pipe *p, void *dst_host, const void *src_device, size_t bytes) {
    ok(cct_hip_pipe_download(p, dst_host, src_device, bytes), "pipe_download");
  }
  void pipe_finish(cct_hip_pipe *p) { ok(cct_hip_pipe_finish(p), "pipe_finish"); }

  // ---- lowering / lifting (DeviceDriver.h:100-122) ----
  void lower_cube(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const PMapHelper args) {
    ok(cct_hip_lower_cube((float *)dst->ptr, (const float *)src->ptr, &args), "lower_cube");
  }
  // pmap2d_read_coalesce<_fpmap_id,_fmap_remap>
  void pmap2d_read_coalesce_remap(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const PMapHelper args) {
    ok(cct_hip_remap((float *)dst->ptr, (const float *)src->ptr, &args), "remap");
  }
  // the backward remap of a convolution together with its bias gradient (one pass over the tensor)
  void pmap2d_read_coalesce_remap_bias_backward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src,
                                                const PMapHelper args, DeviceMemoryPointer *bias) {
    ok(cct_hip_remap_bias_backward((float *)dst->ptr, (const float *)src->ptr, &args, (float *)bias->ptr),
       "remap_bias_backward");
  }
  void inverse_lower_cube(DeviceMemoryPointer *dst, DeviceMemoryPointer *src,
                          const _inverse_lower_cube_arg_helper args) {
    ok(cct_hip_inverse_lower_cube((float *)dst->ptr, (const float *)src->ptr, &args), "inverse_lower_cube");
  }
  void inverse_lower_cube_bias_backward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src,
                                        const _inverse_lower_cube_arg_helper args, DeviceMemoryPointer *bias,
                                        DeviceMemoryPointer *out_grad, int fmap_size, int depth, int batch_size) {
    ok(cct_hip_inverse_lower_cube_bias_backward((float *)dst->ptr, (const float *)src->ptr, &args,
                                                (float *)bias->ptr, (const float *)out_grad->ptr, fmap_size,
                                                depth, batch_size),
       "inverse_lower_cube_bias_backward");
  }

  // ---- bias (DeviceDriver.h:124-138) ----
  void forward_bias(DeviceMemoryPointer *bias, DeviceMemoryPointer *output, const int fmap_size,
                    const int depth, const int batch_size) {
    ok(cct_hip_forward_bias((const float *)bias->ptr, (float *)output->ptr, fmap_size, depth, batch_size),
       "forward_bias");
  }
  void backward_bias(DeviceMemoryPointer *bias, DeviceMemoryPointer *output, const int fmap_size,
                     const int depth, const int batch_size, const float *const device_ones = nullptr) {
    (void)device_ones;  // the reference's gemv-with-ones vector is not needed
    ok(cct_hip_backward_bias((float *)bias->ptr, (const float *)output->ptr, fmap_size, depth, batch_size),
       "backward_bias");
  }
  void backward_bias_fc(DeviceMemoryPointer *bias, DeviceMemoryPointer *output, const int D, const int B,
                        const float *const device_ones = nullptr) {
    (void)device_ones;
    ok(cct_hip_backward_bias_fc((float *)bias->ptr, (const float *)output->ptr, D, B), "backward_bias_fc");
  }

  // ---- pooling / LRN (DeviceDriver.h:140-156) ----
  void lrn_forward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const _lrn_forward_arg_helper args,
                   const _lrn_forward_normalize_arg_helper args2) {
    // argument order as the reference's call site: (input, output) -- LRNBridge_impl.hxx:103
    ok(cct_hip_lrn_forward((float *)src->ptr, (const float *)dst->ptr, &args, &args2), "lrn_forward");
  }
  void lrn_backward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const _lrn_backward_arg_helper args) {
    // (input_grad, output_grad) -- LRNBridge_impl.hxx:168
    ok(cct_hip_lrn_backward((float *)dst->ptr, (const float *)src->ptr, &args), "lrn_backward");
  }
  void maxpool_forward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const _pool_forward_arg_helper args) {
    ok(cct_hip_maxpool_forward((float *)dst->ptr, (const float *)src->ptr, &args), "maxpool_forward");
  }
  void maxpool_backward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const _pool_backward_arg_helper args) {
    // (output_grad, input_grad) -- CPUDriver::maxpool_backward reads dst and writes src
    ok(cct_hip_maxpool_backward((float *)src->ptr, (const float *)dst->ptr, &args), "maxpool_backward");
  }
  // the same followed by the backward of an in-place ReLU on the pooled tensor `relu_data`
  void maxpool_backward_relu(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const _pool_backward_arg_helper args,
                             const float *relu_data) {
    ok(cct_hip_maxpool_backward_relu((float *)src->ptr, (const float *)dst->ptr, &args, relu_data),
       "maxpool_backward_relu");
  }

  // the same from the pooling layer's output tensor (a quarter of the bytes): see cct_hip.h
  void maxpool_backward_relu_pooled(DeviceMemoryPointer *dst, DeviceMemoryPointer *src,
                                    const _pool_backward_arg_helper args, const float *pooled) {
    ok(cct_hip_maxpool_backward_relu_pooled((float *)src->ptr, (const float *)dst->ptr, &args, pooled),
       "maxpool_backward_relu_pooled");
  }

  // ---- the parallel_map pairs of the reference, by name ----
  void relu_forward(DeviceMemoryPointer *dst, DeviceMemoryPointer *src) {
    ok(cct_hip_relu_forward((float *)dst->ptr, (const float *)src->ptr, src->size_in_byte / sizeof(float)),
       "relu_forward");
  }
  void relu_backward(DeviceMemoryPointer *in_grad, DeviceMemoryPointer *out_grad, const float *input_data) {
    ok(cct_hip_relu_backward((float *)in_grad->ptr, (const float *)out_grad->ptr, input_data,
                             out_grad->size_in_byte / sizeof(float)),
       "relu_backward");
  }
  void dropout_forward_train(DeviceMemoryPointer *dst, DeviceMemoryPointer *src, const unsigned int *mask,
                             float scale, unsigned int threshold) {
    ok(cct_hip_dropout_forward_train((float *)dst->ptr, (const float *)src->ptr, mask, scale, threshold,
                                     src->size_in_byte / sizeof(float)),
       "dropout_forward_train");
  }
  void softmax_loss_forward(float *prob, const float *in, const float *labels, float *loss_sum,
                            int len_per_image, int batch) {
    ok(cct_hip_softmax_loss_forward(prob, in, labels, loss_sum, len_per_image, batch), "softmax_loss_forward");
  }
  // forward and backward in one launch (a training iteration asks for both)
  void softmax_loss_forward_backward(float *prob, float *in_grad, const float *in, const float *labels,
                                     float *loss_sum, int len_per_image, int batch, int spatial) {
    ok(cct_hip_softmax_loss_forward_backward(prob, in_grad, in, labels, loss_sum, len_per_image, batch, spatial),
       "softmax_loss_forward_backward");
  }
  void softmax_loss_backward(float *in_grad, const float *prob, const float *labels, int len_per_image,
                             int batch, int spatial) {
    ok(cct_hip_softmax_loss_backward(in_grad, prob, labels, len_per_image, batch, spatial),
       "softmax_loss_backward");
  }

  // ---- single precision BLAS-shaped members (DeviceDriver.h:197-215) ----
  void math_saxpy(const float alpha, DeviceMemoryPointer *X, DeviceMemoryPointer *Y) const {
    ok(cct_hip_math_saxpy(X->size_in_byte / sizeof(float), alpha, (const float *)X->ptr, (float *)Y->ptr),
       "math_saxpy");
  }
  void math_saxpy(const int nItems, const float alpha, float *X, float *Y) const {
    ok(cct_hip_math_saxpy((size_t)nItems, alpha, X, Y), "math_saxpy");
  }
  void math_saxpby(const float alpha, DeviceMemoryPointer *X, const float beta, DeviceMemoryPointer *Y) const {
    ok(cct_hip_math_saxpby(X->size_in_byte / sizeof(float), alpha, (const float *)X->ptr, beta, (float *)Y->ptr),
       "math_saxpby");
  }
  void math_saxpby(const int N, const float alpha, const float *X, const float beta, float *Y) const {
    ok(cct_hip_math_saxpby((size_t)N, alpha, X, beta, Y), "math_saxpby");
  }
  void L1_update(const int n_elements, float *const p_gradient, const float lambda, const float *const p_model) {
    ok(cct_hip_L1_update(n_elements, p_gradient, lambda, p_model), "L1_update");
  }
  void sgd_update(size_t n, float *model, float *gradient, float *history, float stepsize, float momentum,
                  float lambda, bool l1) {
    if (defer_sgd_) {
      cct_sgd_job job = {n, model, gradient, history, stepsize, momentum, lambda, l1 ? 1 : 0};
      std::lock_guard<std::mutex> lk(sgd_mu_);
      sgd_jobs_.push_back(job);
      return;
    }
    ok(cct_hip_sgd_update(n, model, gradient, history, stepsize, momentum, lambda, l1 ? 1 : 0), "sgd_update");
  }
  // Between begin_deferred_sgd() and flush_deferred_sgd() the updates are collected instead of
  // launched (a whole network's backward pass: no layer reads another layer's weights in it);
  // the flush applies the large tensors one launch each and all small ones together.
  void begin_deferred_sgd() {
    static const bool off = [] { const char *e = std::getenv("CCT_HIP_SGD_BATCH"); return e && std::atoi(e) == 0; }();
    defer_sgd_ = !off;  // (tuning override, read once: CCT_HIP_SGD_BATCH=0 keeps one launch per tensor)
  }
  void flush_deferred_sgd() {
    defer_sgd_ = false;
    std::vector<cct_sgd_job> jobs, small;
    {
      std::lock_guard<std::mutex> lk(sgd_mu_);
      jobs.swap(sgd_jobs_);
    }
    for (const cct_sgd_job &j : jobs) {
      if (j.n >= kLargeSgdTensor)
        ok(cct_hip_sgd_update(j.n, j.model, j.gradient, j.history, j.stepsize, j.momentum, j.lambda, j.l1),
           "sgd_update");
      else
        small.push_back(j);
    }
    if (!small.empty()) ok(cct_hip_sgd_update_batch(small.data(), (int)small.size()), "sgd_update_batch");
  }
  // DeviceDriver.h:262-264: X -= Y
  void smath_apply_grad(DeviceMemoryPointer *X, DeviceMemoryPointer *Y) { math_saxpy(-1.0f, Y, X); }
  // CPUDriver forwards this to openblas_set_num_threads (DeviceDriver_CPU.cpp:535-545); a device
  // GEMM has no host thread count, so the call is accepted and ignored
  void set_num_threads(const int) {}
  void sgemm(const enum CBLAS_ORDER order, CBLAS_TRANSPOSE TA, CBLAS_TRANSPOSE TB, int M, int N, int K,
             float alpha, float *pA, int LDA, float *pB, int LDB, float beta, float *pC, int LDC) {
    ok(cct_hip_sgemm(order, TA, TB, M, N, K, alpha, pA, LDA, pB, LDB, beta, pC, LDC), "sgemm");
  }
  void sgemm_new(const CBLAS_TRANSPOSE TA, const CBLAS_TRANSPOSE TB, const int M, const int N, const int K,
                 const float alpha, const float *pA, const float *pB, const float beta, float *pC) {
    ok(cct_hip_sgemm_new(TA, TB, M, N, K, alpha, pA, pB, beta, pC), "sgemm_new");
  }
  // sgemm_new, and beside it the column sums of a rows x cols matrix (an inner-product layer's bias gradient)
  void sgemm_new_colsum(const CBLAS_TRANSPOSE TA, const CBLAS_TRANSPOSE TB, const int M, const int N, const int K,
                        const float alpha, const float *pA, const float *pB, const float beta, float *pC,
                        float *colsum, const float *colsum_src, int rows, int cols) {
    ok(cct_hip_sgemm_new_colsum(TA, TB, M, N, K, alpha, pA, pB, beta, pC, colsum, colsum_src, rows, cols),
       "sgemm_new_colsum");
  }
  // sgemm_new with a bias per column of C and, optionally, the clamp of a following ReLU in the same pass
  void sgemm_new_bias(const CBLAS_TRANSPOSE TA, const CBLAS_TRANSPOSE TB, const int M, const int N, const int K,
                      const float alpha, const float *pA, const float *pB, const float beta, float *pC,
                      const float *col_bias, bool relu = false) {
    ok(cct_hip_sgemm_new_bias(TA, TB, M, N, K, alpha, pA, pB, beta, pC, col_bias, relu ? 1 : 0), "sgemm_new_bias");
  }
  void sgemm_conv_forward(int o, int batch, int fmap, int K, const float *model, const float *lowered,
                          const float *bias, float *out, bool relu = false) {
    ok(cct_hip_sgemm_conv_forward(o, batch, fmap, K, model, lowered, bias, out, relu ? 1 : 0), "sgemm_conv_forward");
  }
  // ---- stride-1 convolution without the lowered matrix (no counterpart in DeviceDriver.h) ----
  // ---- inner-product layers with few outputs (no counterpart in DeviceDriver.h) ----
  bool fc_small_supported(int batch, int in_features, int out_features) {
    return cct_hip_fc_small_supported(batch, in_features, out_features) != 0;
  }
  void fc_small_forward(float *y, const float *x, const float *w, const float *bias, int batch, int in_features,
                        int out_features, bool relu) {
    ok(cct_hip_fc_small_forward(y, x, w, bias, batch, in_features, out_features, relu ? 1 : 0), "fc_small_forward");
  }
  void fc_small_backward(float *dx, float *dw, float *db, const float *dy, const float *x, const float *w, int batch,
                         int in_features, int out_features, const float *relu_data) {
    ok(cct_hip_fc_small_backward(dx, dw, db, dy, x, w, batch, in_features, out_features, relu_data),
       "fc_small_backward");
  }
  // ---- convolutions with a very short contraction and few maps (no counterpart in DeviceDriver.h) ----
  bool conv_small_supported(int batch, int depth, int n, int k, int stride, int padding, int num_outputs) {
    return cct_hip_conv_small_supported(batch, depth, n, k, stride, padding, num_outputs) != 0;
  }
  void conv_small_forward(float *out, const float *in, const float *model, const float *bias, int batch, int depth,
                          int n, int k, int padding, int num_outputs, bool relu) {
    ok(cct_hip_conv_small_forward(out, in, model, bias, batch, depth, n, k, padding, num_outputs, relu ? 1 : 0),
       "conv_small_forward");
  }
  void conv_small_backward_weights(float *dw, float *db, const float *dout, const float *in, int batch, int depth,
                                   int n, int k, int padding, int num_outputs) {
    ok(cct_hip_conv_small_backward_weights(dw, db, dout, in, batch, depth, n, k, padding, num_outputs),
       "conv_small_backward_weights");
  }
  // ---- 1 x 1 convolutions: products on the tensors as they lie (no counterpart in DeviceDriver.h) ----
  bool conv1x1_supported(int batch, int depth, int n, int k, int stride, int padding, int num_outputs) {
    return cct_hip_conv1x1_supported(batch, depth, n, k, stride, padding, num_outputs) != 0;
  }
  void conv1x1_forward(float *out, const float *in, const float *model, const float *bias, int batch, int depth,
                       int plane, int num_outputs, bool relu) {
    ok(cct_hip_conv1x1_forward(out, in, model, bias, batch, depth, plane, num_outputs, relu ? 1 : 0), "conv1x1_forward");
  }
  void conv1x1_backward_data(float *din, const float *dout, const float *model, int batch, int depth, int plane,
                             int num_outputs) {
    ok(cct_hip_conv1x1_backward_data(din, dout, model, batch, depth, plane, num_outputs), "conv1x1_backward_data");
  }
  void conv1x1_backward_weights(float *dw, float *db, const float *dout, const float *in, int batch, int depth,
                                int plane, int num_outputs) {
    ok(cct_hip_conv1x1_backward_weights(dw, db, dout, in, batch, depth, plane, num_outputs), "conv1x1_backward_weights");
  }
  // `groups` > 1: a grouped convolution (depth and num_outputs are the layer's totals), all groups in one launch
  bool conv_direct_supported(int batch, int depth, int n, int k, int stride, int padding, int num_outputs,
                             int groups = 1) {
    return cct_hip_conv_direct_supported_grouped(batch, depth, n, k, stride, padding, num_outputs, groups) != 0;
  }
  size_t conv_direct_slab_floats(int num_outputs, int depth, int k, int for_data_gradient, int groups = 1) {
    return cct_hip_conv_direct_slab_floats_grouped(num_outputs, depth, k, for_data_gradient, groups);
  }
  void conv_direct_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                         int for_data_gradient, int groups = 1) {
    ok(cct_hip_conv_direct_slabs_grouped(slabs, model, num_outputs, depth, k, for_data_gradient, groups),
       "conv_direct_slabs");
  }
  void conv_direct_forward(float *output, const float *input, const float *slabs, const float *bias, int batch,
                           int depth, int n, int k, int padding, int num_outputs, size_t in_stride = 0,
                           size_t out_stride = 0, bool relu = false, int groups = 1) {
    ok(cct_hip_conv_direct_forward_grouped(output, input, slabs, bias, batch, depth, n, k, padding, num_outputs,
                                           in_stride, out_stride, relu ? 1 : 0, groups),
       "conv_direct_forward");
  }
  // relu_data (optional): the layer's input tensor when it is the output of an in-place ReLU -- the
  // gradient is then stored already masked with (relu_data > 0)
  void conv_direct_backward_data(float *input_grad, const float *output_grad, const float *slabs, int batch,
                                 int depth, int n, int k, int padding, int num_outputs, size_t in_stride = 0,
                                 size_t out_stride = 0, const float *relu_data = nullptr, int groups = 1) {
    ok(cct_hip_conv_direct_backward_data_grouped(input_grad, output_grad, slabs, batch, depth, n, k, padding,
                                                 num_outputs, in_stride, out_stride, relu_data, groups),
       relu_data ? "conv_direct_backward_data_relu" : "conv_direct_backward_data");
  }
  void conv_direct_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                    const float *input, int batch, int depth, int n, int k, int padding,
                                    int num_outputs, size_t in_stride = 0, size_t out_stride = 0, int groups = 1) {
    ok(cct_hip_conv_direct_backward_weights_grouped(model_grad, bias_grad, output_grad, input, batch, depth, n, k,
                                                    padding, num_outputs, in_stride, out_stride, groups),
       "conv_direct_backward_weights");
  }
  // ---- strided convolution without the lowered matrix (no counterpart in DeviceDriver.h) ----
  bool conv_strided_supported(int batch, int depth, int n, int k, int stride, int padding, int num_outputs) {
    return cct_hip_conv_strided_supported(batch, depth, n, k, stride, padding, num_outputs) != 0;
  }
  size_t conv_strided_slab_floats(int num_outputs, int depth, int k, int stride, int padding) {
    return cct_hip_conv_strided_slab_floats(num_outputs, depth, k, stride, padding);
  }
  void conv_strided_slabs(float *slabs, const float *model, int num_outputs, int depth, int k, int stride,
                          int padding) {
    ok(cct_hip_conv_strided_slabs(slabs, model, num_outputs, depth, k, stride, padding), "conv_strided_slabs");
  }
  void conv_strided_forward(float *output, const float *input, const float *slabs, const float *bias, int batch,
                            int depth, int n, int k, int stride, int padding, int num_outputs, bool relu = false) {
    ok(cct_hip_conv_strided_forward(output, input, slabs, bias, batch, depth, n, k, stride, padding, num_outputs,
                                    relu ? 1 : 0),
       "conv_strided_forward");
  }
  void conv_strided_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                     const float *input, int batch, int depth, int n, int k, int stride,
                                     int padding, int num_outputs) {
    ok(cct_hip_conv_strided_backward_weights(model_grad, bias_grad, output_grad, input, batch, depth, n, k, stride,
                                             padding, num_outputs),
       "conv_strided_backward_weights");
  }
  bool conv_strided_backward_data_supported(int batch, int depth, int n, int k, int stride, int padding,
                                            int num_outputs) {
    return cct_hip_conv_strided_backward_data_supported(batch, depth, n, k, stride, padding, num_outputs) != 0;
  }
  size_t conv_strided_backward_data_slab_floats(int num_outputs, int depth, int k, int stride) {
    return cct_hip_conv_strided_backward_data_slab_floats(num_outputs, depth, k, stride);
  }
  void conv_strided_backward_data_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                                        int stride) {
    ok(cct_hip_conv_strided_backward_data_slabs(slabs, model, num_outputs, depth, k, stride),
       "conv_strided_backward_data_slabs");
  }
  void conv_strided_backward_data(float *input_grad, const float *output_grad, const float *slabs, int batch,
                                  int depth, int n, int k, int stride, int padding, int num_outputs) {
    ok(cct_hip_conv_strided_backward_data(input_grad, output_grad, slabs, batch, depth, n, k, stride, padding,
                                          num_outputs),
       "conv_strided_backward_data");
  }
  void sgemv(const CBLAS_TRANSPOSE TA, const int M, const int N, const float alpha, const float *pA,
             const float *px, const float beta, float *py) {
    ok(cct_hip_sgemv(TA, M, N, alpha, pA, px, beta, py), "sgemv");
  }

  // ---- fillers / rng (DeviceDriver.h:238-260) ----
  void init_rng(const int random_seed) { ok(cct_hip_init_rng(random_seed), "init_rng"); }
  void rand_uint_initialize(unsigned int *buf, const int n) {
    ok(cct_hip_rand_uint_initialize(buf, n), "rand_uint_initialize");
  }
  // Random fillers: host draws from std::mt19937 with the same distributions and call order as
  // CPUDriver (src/sched/DeviceDriver_CPU.cpp:661-699), copied to the device by the library.
  void sinitialize_xavier(DeviceMemoryPointer *arr, const size_t n_batch, const int random_seed = -1) {
    ok(cct_hip_fill_xavier((float *)arr->ptr, arr->size_in_byte / sizeof(float), n_batch, random_seed),
       "sinitialize_xavier");
  }
  void sbernoulli_initialize(DeviceMemoryPointer *arr, const float p, const int random_seed = -1) {
    ok(cct_hip_fill_bernoulli((float *)arr->ptr, arr->size_in_byte / sizeof(float), p, random_seed),
       "sbernoulli_initialize");
  }
  void sgaussian_initialize(DeviceMemoryPointer *arr, const float mean, const float std_dev,
                            const int random_seed = -1) {
    ok(cct_hip_fill_gaussian((float *)arr->ptr, arr->size_in_byte / sizeof(float), mean, std_dev, random_seed),
       "sgaussian_initialize");
  }
  void sconstant_initialize(DeviceMemoryPointer *arr, const float value) {
    ok(cct_hip_sconstant_initialize((float *)arr->ptr, arr->size_in_byte / sizeof(float), value),
       "sconstant_initialize");
  }

  // ---- hooks (DeviceDriver.h:266-272) ----
  void device_sync() { ok(cct_hip_device_sync(), "device_sync"); }
  void init_thread() { ok(cct_hip_init(device_id_), "init_thread"); }
  void destroy_thread() {}
  void set_device_id(int id) { device_id_ = id; ok(cct_hip_init(id), "set_device_id"); }

 private:
  int device_id_ = 0;
  static void ok(int rc, const char *what) {
    if (rc != 0)
      host_fail(std::string("HIPDriver::") + what + " failed (" + std::to_string(rc) + "): " + cct_hip_last_error());
  }

 private:
  static constexpr size_t kLargeSgdTensor = (size_t)1 << 20;  // elements; above this a launch of its own pays
  bool defer_sgd_ = false;
  std::mutex sgd_mu_;
  std::vector<cct_sgd_job> sgd_jobs_;
};

}  // namespace cct
