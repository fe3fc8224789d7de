// Convolution operator for the HIP driver: lowering -> GEMM -> (remap, bias) forward;
// bias gradient, data-gradient GEMM -> lifting, weight-gradient GEMM backward.
//
// Counterpart of ConvolutionBridge<float, Layout_CRDB, float, Layout_CRDB, DriverClass>
// (src/bridges/ConvolutionBridge.h:74-215, _impl.hxx:13-226, 284-520, 541-796).  It follows the
// reference's *batched* branch (the one CPUDriver takes, _impl.hxx:294-373 and 551-628): the
// whole batch is lowered once into a (k*k*d) x (m*m*b) buffer that the backward pass reuses,
// rather than the per-image loop the reference runs for non-CPU drivers (:375-520, 630-796).
// Deliberate departures, none of which changes a result:
//   * the output-gradient cube is permuted into a scratch cube, not in place (:604);
//   * by default the forward GEMM writes [b][o][m*m] and adds the bias in its epilogue instead
//     of running remap_output and the bias map as separate passes (set_fused(false) restores
//     the staged sequence);
//   * the bias gradient is reduced in the same launch as the lifting kernel;
//   * for stride-1 layers with k = 3, 5 or 7 the data gradient (path level 2) or all three products
//     (level 3, the default where the geometry allows it) come from direct-convolution kernels
//     that never materialise the lowered matrices; results then agree with the lowering path to
//     fp32 rounding instead of bit for bit.  The lowered buffers are allocated on first use, so
//     level 3 runs without them;
//   * strided layers with k = 11 (stride 4) or k = 7, 5, 3 (stride 2) take level 3 with direct forward
//     and weight-gradient kernels of their own; their data gradient (not needed for a first layer)
//     comes from a direct kernel too where it covers the geometry (depth * stride^2 <= 80 in an odd
//     number of 16-row blocks: AlexNet / CaffeNet conv1), else from the data-gradient GEMM and the
//     lifting, which need no lowered input;
//   * `group` > 1 (cnn.proto ConvolutionParameter.group, which the reference's bridge ignores and its
//     network builder realises as towers between a Split and a Concat, src/DeepNet.h:1700-1757) is
//     run by this one bridge: the model cube is [o][d/group][k][k] (the blob layout Caffe gives such
//     a layer), group q maps its slice of the input channels to its slice of the output maps, and the
//     direct kernels run all groups in one launch each.  Only the all-direct path covers it;
//   * stride-1 layers with one or three input channels, k = 3 or 5 and at most 32 maps (LeNet's first
//     layer) take plain multiply-add kernels for the forward pass and the weight gradient where they
//     would take the all-direct path (set_small_kernels): the forward launch reads the model cube as it
//     is, so no slabs are built for it;
//   * 1 x 1 layers (stride 1, no padding) take level 3 as products on the tensors as they lie: lowering such a
//     layer is a permuting copy, and so are the remap and the lifting.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <string>

#include "AbstractBridge.h"
#include "Connector.h"
#include "Kernel.h"

namespace cct {

// How much of the lowering pipeline is replaced (set_path).
enum ConvPath {
  PATH_STAGED = 0,       // the reference's sequence of separate passes
  PATH_FUSED = 1,        // GEMM epilogue does remap + bias; bias gradient rides with the lifting
  PATH_DIRECT_DATA = 2,  // as 1, data gradient by the direct kernel (no data-gradient GEMM, no lifting)
  PATH_DIRECT_ALL = 3    // forward, weight gradient and data gradient by direct kernels, no lowering
};

// GEMM size (FLOP) from which a layer takes the all-direct path by default.
constexpr double kConvDirectMinFlop = 2e9;

// Stage labels of the reference's detailed profiling output (_impl.hxx:325-366, 601-623).
enum ConvStage {
  STAGE_LOWER = 0, STAGE_GEMM, STAGE_REMAP, STAGE_BIAS,            // forward
  STAGE_BW_BIAS, STAGE_BW_REMAP, STAGE_GEMM_DATA, STAGE_INVERSE_LOWER, STAGE_GEMM_WEIGHTS,  // backward
  STAGE_COUNT
};

template <typename DataType, typename DriverClass>
class ConvolutionBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  using Base::iR; using Base::iC; using Base::iD; using Base::iB;
  using Base::oR; using Base::oC; using Base::oD; using Base::oB;
  using Base::needs_to_calc_backward_grad;
  using Base::layer_param; using Base::solver_param; using Base::p_driver;
  using Base::p_input_layer; using Base::p_output_layer;
  using Base::report_forward_history; using Base::report_backward_updateweight_history;
  typedef Layer<DataType> InputLayerType;
  typedef Layer<DataType> OutputLayerType;
  typedef LogicalCube<DataType> LogicalCubeType;

  const size_t K;
  const size_t group;  // channel groups (1: an ordinary convolution)
  const size_t num_output_features;
  const size_t stride;
  const size_t padding;
  const bool bias_term;
  const cnn::FillerParameter weight_filler;
  const cnn::FillerParameter bias_filler;

  LogicalCubeType *p_model_cube;  // [o][d][k][k] == GEMM matrix [o x k*k*d]
  LogicalCubeType *p_bias_cube;   // [o]

  ConvolutionBridge(InputLayerType *const _p_input_layer, OutputLayerType *const _p_output_layer,
                    const cnn::LayerParameter *const _layer_param,
                    const cnn::SolverParameter *const _solver_param, DriverClass *const _p_driver)
      : Base(_p_input_layer, _p_output_layer, _layer_param, _solver_param, _p_driver),
        K(_layer_param->convolution_param().kernel_size()),
        group(_layer_param->convolution_param().group() > 1 ? _layer_param->convolution_param().group() : 1),
        num_output_features(_p_output_layer->dD),
        stride(_layer_param->convolution_param().stride()), padding(_layer_param->convolution_param().pad()),
        bias_term(_layer_param->convolution_param().bias_term()),
        weight_filler(_layer_param->convolution_param().weight_filler()),
        bias_filler(_layer_param->convolution_param().bias_filler()), p_model_cube(nullptr),
        p_bias_cube(nullptr), p_bias_gradient_cube(nullptr) {
    if (oR != (iR + 2 * padding - K) / stride + 1 || oC != (iC + 2 * padding - K) / stride + 1 || iB != oB ||
        num_output_features != oD || iR != iC || iD % group || num_output_features % group) {
      host_fail("ConvolutionBridge: inconsistent layer shapes");
    }
    // cubes read outside the bridge (model / gradients), device resident
    p_model_cube = new LogicalCubeType(K, K, iD / group, num_output_features, p_driver);
    initialize_logical_cube(p_model_cube, weight_filler);
    p_model_gradient_cube = new LogicalCubeType(K, K, iD / group, num_output_features, p_driver);
    DeviceMemoryPointer mg = p_model_gradient_cube->get_device_pointer(p_driver);
    p_driver->sconstant_initialize(&mg, DataType(0.));
    if (bias_term) {
      p_bias_cube = new LogicalCubeType(1, 1, num_output_features, 1, p_driver);
      initialize_logical_cube(p_bias_cube, bias_filler);
      p_bias_gradient_cube = new LogicalCubeType(1, 1, num_output_features, 1, p_driver);
      DeviceMemoryPointer bg = p_bias_gradient_cube->get_device_pointer(p_driver);
      p_driver->sconstant_initialize(&bg, DataType(0.));
    }
    // cubes used inside the bridge only, sized for the whole batch, allocated on first use
    p_forward_lowered_data = nullptr;
    p_backward_inputgrad = nullptr;
    p_staging_cube = nullptr;
    p_forward_slabs = nullptr;
    p_backward_slabs = nullptr;

    // shapes of the lowering path's GEMM operands (never run for a grouped layer)
    LogicalCubeType lowered_forward_model(nullptr, num_output_features, K * K * iD, 1, 1);
    LogicalCubeType lowered_forward_output(nullptr, num_output_features, oR * oC * iB, 1, 1);
    LogicalCubeType lowered_data(nullptr, K * K * iD, oR * oC * iB, 1, 1);
    LogicalCubeType dummy_data_cube(nullptr, iR, iC, iD, iB);
    p_forward_lower_connector =
        new Connector<DataType, DriverClass>(&dummy_data_cube, &lowered_data, K, padding, stride, p_driver);
    p_forward_gemm_kernel = new Kernel<DataType, KernelConfig_GEMM_NOTRANS_TRANS_NO_DIM_FLIP, DriverClass>(
        &lowered_forward_model, &lowered_data, &lowered_forward_output, p_driver);
    p_backward_gemm_updateweight_kernel = new Kernel<DataType, KernelConfig_GEMM_NOTRANS_NOTRANS_DIM_FLIP, DriverClass>(
        &lowered_forward_output, &lowered_data, &lowered_forward_model, p_driver);
    p_backward_gemm_updategrad_kernel = new Kernel<DataType, KernelConfig_GEMM_TRANS_NOTRANS, DriverClass>(
        &lowered_forward_model, &lowered_forward_output, &lowered_data, p_driver);
    direct_ok_ = p_driver->conv_direct_supported((int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                                 (int)num_output_features, (int)group);
    if (group > 1 && !direct_ok_)
      host_fail("ConvolutionBridge: a grouped convolution runs on the direct kernels only, which do not cover this geometry");
    // one or three channels and a few maps (LeNet's first layer): plain multiply-add kernels for the forward pass and
    // the weight gradient that read the model cube as it is (no slabs); they run where the all-direct path does
    small_ok_ = direct_ok_ && group == 1 &&
                p_driver->conv_small_supported((int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                               (int)num_output_features);
    strided_ok_ = !direct_ok_ && group == 1 && p_driver->conv_strided_supported((int)iB, (int)iD, (int)iR, (int)K, (int)stride,
                                                                  (int)padding, (int)num_output_features);
    pointwise_ok_ = !direct_ok_ && !strided_ok_ && group == 1 &&
                    p_driver->conv1x1_supported((int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                                (int)num_output_features);
    strided_data_ok_ = strided_ok_ && p_driver->conv_strided_backward_data_supported(
                                          (int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                          (int)num_output_features);
    // Small layers (LeNet-sized) stay on the fused lowering path by default: the direct kernels'
    // fixed costs (slab re-layout, partial-sum reduction) outweigh what they save below a few GFLOP.
    const double gemm_flop = 2.0 * num_output_features * (double)(oR * oC * iB) * (double)(K * K * iD / group);
    // (a very short contraction -- LeNet conv1 has k*k*d = 25 -- makes the lowered GEMM all prologue and
    // epilogue; there the direct kernels win at any size)
    const bool short_contraction = K * K * iD <= 64;
    default_path_ = (direct_ok_ && (gemm_flop >= kConvDirectMinFlop || short_contraction)) ? PATH_DIRECT_ALL : PATH_FUSED;
    if (strided_ok_ && gemm_flop >= kConvDirectMinFlop) default_path_ = PATH_DIRECT_ALL;
    if (pointwise_ok_) default_path_ = PATH_DIRECT_ALL;  // fewer launches and no copies at any size
    if (group > 1) default_path_ = PATH_DIRECT_ALL;
    path_ = default_path_;
    for (int i = 0; i < STAGE_COUNT; ++i) { timers_[i] = nullptr; stage_ms_[i] = 0.f; }
  }

  ~ConvolutionBridge() {
    for (int i = 0; i < STAGE_COUNT; ++i)
      if (timers_[i]) cct_hip_timer_destroy(timers_[i]);
    delete p_model_cube;
    delete p_model_gradient_cube;
    delete p_bias_cube;
    delete p_bias_gradient_cube;
    delete p_forward_lowered_data;
    delete p_backward_inputgrad;
    delete p_staging_cube;
    delete p_forward_slabs;
    delete p_backward_slabs;
    delete p_forward_lower_connector;
    delete p_forward_gemm_kernel;
    delete p_backward_gemm_updateweight_kernel;
    delete p_backward_gemm_updategrad_kernel;
  }

  LogicalCubeType *get_model_cube() override { return p_model_cube; }
  LogicalCubeType *get_bias_cube() override { return p_bias_cube; }
  LogicalCubeType *get_model_grad_cube() override { return p_model_gradient_cube; }
  LogicalCubeType *get_bias_grad_cube() override { return p_bias_gradient_cube; }
  LogicalCubeType *get_lowered_cube() { return lowered(); }

  // Path level (ConvPath); levels 2 and 3 fall back to 1 where the direct kernels do not cover
  // the layer's geometry.
  void set_path(int level) {
    if (level < PATH_STAGED) level = PATH_STAGED;
    if (level > PATH_DIRECT_ALL) level = PATH_DIRECT_ALL;
    if (level >= PATH_DIRECT_DATA && !direct_ok_)
      level = ((strided_ok_ || pointwise_ok_) && level == PATH_DIRECT_ALL) ? PATH_DIRECT_ALL : PATH_FUSED;
    if (views_ || group > 1) level = PATH_DIRECT_ALL;  // the lowering path cannot address channel slices
    path_ = level;
  }
  int path() const { return path_; }
  // True if this geometry runs on the all-direct path by default.
  bool direct_by_default() const { return default_path_ == PATH_DIRECT_ALL; }
  // The layers' cubes are channel slices of wider tensors: `in_stride` / `out_stride` floats lie
  // between consecutive images (0 = dense).  Only the all-direct path can work on such views; the
  // bridge then stays on it.
  void set_image_strides(size_t in_stride, size_t out_stride) {
    if (!direct_ok_) {
      host_fail("ConvolutionBridge: channel-slice views need the direct kernels");
    }
    in_image_stride_ = in_stride;
    out_image_stride_ = out_stride;
    path_ = PATH_DIRECT_ALL;
    views_ = true;
  }
  void set_fused(bool on) { set_path(on ? default_path_ : PATH_STAGED); }
  // The plain multiply-add kernels for layers of one or three channels and few maps, on by default where they
  // apply (on the all-direct path, on dense tensors); off: the MFMA direct kernels run such a layer too.
  void set_small_kernels(bool on) { use_small_ = on; }
  bool small_kernels() const { return small_ok_ && use_small_ && !views_; }
  // Apply the ReLU of a following in-place ReLUBridge (y = max(x, 0)) while the output is stored,
  // instead of in a pass of its own; the ReLU bridge then skips its forward.
  void set_fuse_relu(bool on) { fuse_relu_ = on; }
  // The input layer is the output of an in-place ReLU whose backward this bridge performs on the
  // input gradient it produces (masked in the direct kernel's store, or by a pass after the lifting);
  // the ReLU bridge then skips its own.  Only meaningful with needs_to_calc_backward_grad.
  bool input_is_relu_output = false;
  bool fuse_relu() const { return fuse_relu_; }
  // per-stage hipEvent timing (the reference's -D_DETAILED_PROFILING stage prints)
  void set_stage_profiling(bool on) { profile_ = on; }
  float stage_ms(int stage) {
    float ms = 0.f;
    if (timers_[stage] && stage_ran_[stage]) cct_hip_timer_elapsed_ms(timers_[stage], &ms);
    return ms;
  }
  // the kernel instance the driver chose for the stage's product kernel the last time it ran with
  // stage profiling on ("" if it has not)
  const std::string &stage_kernel(int stage) const { return stage_kernel_[stage]; }

  // ---- the passes on a range of images (for a scheduler that moves the batch in pieces) ----
  // True when forward and data gradient can run on images [b0, b0 + nb) alone: the all-direct path, whose
  // kernels take a batch count and tensor pointers (every image's result is independent of the others; the
  // weight gradient sums over the batch and stays one call over all of it).
  bool supports_batch_ranges() const { return path_ == PATH_DIRECT_ALL && !views_; }
  // once per pass, before the first range: the weight slabs (the model changes between iterations)
  void forward_prepare() {
    if (small_kernels() || pointwise_ok_)
      return;  // these read the model cube itself
    if (strided_ok_)
      p_driver->conv_strided_slabs(forward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                   (int)num_output_features, (int)iD, (int)K, (int)stride, (int)padding);
    else
      p_driver->conv_direct_slabs(forward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                  (int)num_output_features, (int)iD, (int)K, 0, (int)group);
  }
  void forward_range(size_t b0, size_t nb) {
    const size_t in_img = iR * iC * iD, out_img = oR * oC * oD;
    float *out = p_output_layer->p_data_cube->get_p_data() + b0 * out_img;
    const float *in = p_input_layer->p_data_cube->get_p_data() + b0 * in_img;
    const float *bias = bias_term ? p_bias_cube->get_p_data() : nullptr;
    if (pointwise_ok_)
      p_driver->conv1x1_forward(out, in, p_model_cube->get_p_data(), bias, (int)nb, (int)iD, (int)(iR * iC),
                                (int)num_output_features, fuse_relu_);
    else if (small_kernels())
      p_driver->conv_small_forward(out, in, p_model_cube->get_p_data(), bias, (int)nb, (int)iD, (int)iR, (int)K,
                                   (int)padding, (int)num_output_features, fuse_relu_);
    else if (strided_ok_)
      p_driver->conv_strided_forward(out, in, forward_slabs()->get_p_data(), bias, (int)nb, (int)iD, (int)iR, (int)K,
                                     (int)stride, (int)padding, (int)num_output_features, fuse_relu_);
    else
      p_driver->conv_direct_forward(out, in, forward_slabs()->get_p_data(), bias, (int)nb, (int)iD, (int)iR, (int)K,
                                    (int)padding, (int)num_output_features, 0, 0, fuse_relu_, (int)group);
  }
  // data gradient of a range; false if this layer's data gradient is not a per-range kernel (a strided layer
  // without the phase-decomposed kernel): the caller then runs backward() on the whole batch
  bool backward_data_ranges_supported() const {
    return supports_batch_ranges() && (direct_ok_ || strided_data_ok_ || pointwise_ok_);
  }
  void backward_data_prepare() {
    if (pointwise_ok_) return;
    if (direct_ok_)
      p_driver->conv_direct_slabs(backward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                  (int)num_output_features, (int)iD, (int)K, 1, (int)group);
    else
      p_driver->conv_strided_backward_data_slabs(backward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                                 (int)num_output_features, (int)iD, (int)K, (int)stride);
  }
  void backward_data_range(size_t b0, size_t nb) {
    const size_t in_img = iR * iC * iD, out_img = oR * oC * oD;
    float *ig = p_input_layer->p_gradient_cube->get_p_data() + b0 * in_img;
    const float *og = p_output_layer->p_gradient_cube->get_p_data() + b0 * out_img;
    const float *in = p_input_layer->p_data_cube->get_p_data() + b0 * in_img;
    if (pointwise_ok_) {
      p_driver->conv1x1_backward_data(ig, og, p_model_cube->get_p_data(), (int)nb, (int)iD, (int)(iR * iC),
                                      (int)num_output_features);
      if (input_is_relu_output) {
        DeviceMemoryPointer g = p_driver->get_device_pointer(ig, nb * in_img * sizeof(DataType));
        p_driver->relu_backward(&g, &g, in);
      }
    } else if (direct_ok_) {
      p_driver->conv_direct_backward_data(ig, og, backward_slabs()->get_p_data(), (int)nb, (int)iD, (int)iR, (int)K,
                                          (int)padding, (int)num_output_features, 0, 0,
                                          input_is_relu_output ? in : nullptr, (int)group);
    } else {
      p_driver->conv_strided_backward_data(ig, og, backward_slabs()->get_p_data(), (int)nb, (int)iD, (int)iR, (int)K,
                                           (int)stride, (int)padding, (int)num_output_features);
      if (input_is_relu_output) {
        DeviceMemoryPointer g = p_driver->get_device_pointer(ig, nb * in_img * sizeof(DataType));
        p_driver->relu_backward(&g, &g, in);
      }
    }
  }
  // weight and bias gradient over the whole batch (all-direct path)
  void backward_weights_all() {
    float *dw = p_model_gradient_cube->get_p_data();
    float *db = bias_term ? p_bias_gradient_cube->get_p_data() : nullptr;
    const float *og = p_output_layer->p_gradient_cube->get_p_data();
    const float *in = p_input_layer->p_data_cube->get_p_data();
    if (pointwise_ok_)
      p_driver->conv1x1_backward_weights(dw, db, og, in, (int)iB, (int)iD, (int)(iR * iC), (int)num_output_features);
    else if (small_kernels())
      p_driver->conv_small_backward_weights(dw, db, og, in, (int)iB, (int)iD, (int)iR, (int)K, (int)padding,
                                            (int)num_output_features);
    else if (strided_ok_)
      p_driver->conv_strided_backward_weights(dw, db, og, in, (int)iB, (int)iD, (int)iR, (int)K, (int)stride,
                                              (int)padding, (int)num_output_features);
    else
      p_driver->conv_direct_backward_weights(dw, db, og, in, (int)iB, (int)iD, (int)iR, (int)K, (int)padding,
                                             (int)num_output_features, 0, 0, (int)group);
  }

  // (1) input --lowering--> lowered  (2) model x lowered^T --> output  (3) remap + bias
  void forward() override {
    report_forward_history.reset();
    for (int i = STAGE_LOWER; i <= STAGE_BIAS; ++i) { stage_ran_[i] = false; if (profile_) stage_kernel_[i].clear(); }
    LogicalCubeType *input_d_cube = p_input_layer->p_data_cube;
    LogicalCubeType *output_d_cube = p_output_layer->p_data_cube;
    LogicalCubeType lowered_model(p_model_cube->get_p_data(), num_output_features, K * K * iD, 1, 1);

    if (path_ == PATH_DIRECT_ALL && strided_ok_) {
      begin(STAGE_GEMM);
      p_driver->conv_strided_slabs(forward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                   (int)num_output_features, (int)iD, (int)K, (int)stride, (int)padding);
      p_driver->conv_strided_forward(output_d_cube->get_p_data(), input_d_cube->get_p_data(),
                                     forward_slabs()->get_p_data(), bias_term ? p_bias_cube->get_p_data() : nullptr,
                                     (int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                     (int)num_output_features, fuse_relu_);
      end(STAGE_GEMM);
      report_forward_history.end();
      return;
    }
    if (path_ == PATH_DIRECT_ALL && pointwise_ok_) {
      begin(STAGE_GEMM);
      p_driver->conv1x1_forward(output_d_cube->get_p_data(), input_d_cube->get_p_data(), p_model_cube->get_p_data(),
                                bias_term ? p_bias_cube->get_p_data() : nullptr, (int)iB, (int)iD, (int)(iR * iC),
                                (int)num_output_features, fuse_relu_);
      end(STAGE_GEMM);
      report_forward_history.end();
      return;
    }
    if (path_ == PATH_DIRECT_ALL && small_kernels()) {
      begin(STAGE_GEMM);
      p_driver->conv_small_forward(output_d_cube->get_p_data(), input_d_cube->get_p_data(), p_model_cube->get_p_data(),
                                   bias_term ? p_bias_cube->get_p_data() : nullptr, (int)iB, (int)iD, (int)iR, (int)K,
                                   (int)padding, (int)num_output_features, fuse_relu_);
      end(STAGE_GEMM);
      report_forward_history.end();
      return;
    }
    if (path_ == PATH_DIRECT_ALL) {
      // slabs are rebuilt every pass: the model changes between iterations
      begin(STAGE_GEMM);
      p_driver->conv_direct_slabs(forward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                  (int)num_output_features, (int)iD, (int)K, 0, (int)group);
      p_driver->conv_direct_forward(output_d_cube->get_p_data(), input_d_cube->get_p_data(),
                                    forward_slabs()->get_p_data(), bias_term ? p_bias_cube->get_p_data() : nullptr,
                                    (int)iB, (int)iD, (int)iR, (int)K, (int)padding, (int)num_output_features,
                                    in_image_stride_, out_image_stride_, fuse_relu_, (int)group);
      end(STAGE_GEMM);
      report_forward_history.end();
      return;
    }
    begin(STAGE_LOWER);
    p_forward_lower_connector->lower_cube(input_d_cube, lowered());
    end(STAGE_LOWER);
    if (path_ >= PATH_FUSED) {
      begin(STAGE_GEMM);
      p_driver->sgemm_conv_forward((int)num_output_features, (int)iB, (int)(oR * oC), (int)(K * K * iD),
                                   p_model_cube->get_p_data(), lowered()->get_p_data(),
                                   bias_term ? p_bias_cube->get_p_data() : nullptr, output_d_cube->get_p_data(),
                                   fuse_relu_);
      end(STAGE_GEMM);
    } else {
      LogicalCubeType lowered_output(staging()->get_p_data(), num_output_features, oR * oC * iB, 1, 1);
      begin(STAGE_GEMM);
      p_forward_gemm_kernel->compute(&lowered_model, lowered(), &lowered_output);
      end(STAGE_GEMM);
      begin(STAGE_REMAP);
      p_forward_lower_connector->remap_output(*output_d_cube, *staging(), num_output_features, iB);
      end(STAGE_REMAP);
      if (bias_term) {
        begin(STAGE_BIAS);
        DeviceMemoryPointer output = output_d_cube->get_device_pointer(p_driver);
        DeviceMemoryPointer bias = p_bias_cube->get_device_pointer(p_driver);
        p_driver->forward_bias(&bias, &output, (int)(oR * oC), (int)oD, (int)iB);
        end(STAGE_BIAS);
      }
      if (fuse_relu_) {  // the staged sequence has no epilogue to fold it into
        DeviceMemoryPointer output = output_d_cube->get_device_pointer(p_driver);
        p_driver->relu_forward(&output, &output);
      }
    }
    report_forward_history.end();
  }

  // bias gradient; remap of the output gradient; data-gradient GEMM + lifting (if needed);
  // weight-gradient GEMM against the lowered data kept from forward()
  void backward() override {
    report_backward_updateweight_history.reset();
    for (int i = STAGE_BW_BIAS; i < STAGE_COUNT; ++i) { stage_ran_[i] = false; if (profile_) stage_kernel_[i].clear(); }
    LogicalCubeType *output_g_cube = p_output_layer->p_gradient_cube;
    LogicalCubeType *input_g_cube = p_input_layer->p_gradient_cube;
    LogicalCubeType lowered_model(p_model_cube->get_p_data(), num_output_features, K * K * iD, 1, 1);
    LogicalCubeType lowered_model_grad(p_model_gradient_cube->get_p_data(), num_output_features, K * K * iD, 1, 1);
    DeviceMemoryPointer og = output_g_cube->get_device_pointer(p_driver);
    if (path_ == PATH_DIRECT_ALL && pointwise_ok_) {
      begin(STAGE_GEMM_WEIGHTS);
      backward_weights_all();
      end(STAGE_GEMM_WEIGHTS);
      if (needs_to_calc_backward_grad) {
        begin(STAGE_GEMM_DATA);
        backward_data_range(0, iB);
        end(STAGE_GEMM_DATA);
      }
      report_backward_updateweight_history.end();
      return;
    }
    const bool direct_data = path_ >= PATH_DIRECT_DATA && needs_to_calc_backward_grad && direct_ok_;
    const bool direct_weights = path_ == PATH_DIRECT_ALL;
    // a strided layer on the all-direct path that must hand back an input gradient: the permuted output
    // gradient feeds the data-gradient GEMM, whose result is lifted (neither needs the lowered input)
    const bool strided_direct_data = direct_weights && strided_data_ok_ && needs_to_calc_backward_grad;
    const bool strided_data = direct_weights && strided_ok_ && needs_to_calc_backward_grad && !strided_direct_data;

    const bool fuse_bias_into_lift = bias_term && needs_to_calc_backward_grad && path_ == PATH_FUSED;
    // on the all-direct path the weight-gradient kernel reduces the bias gradient as well
    // a layer without an input gradient has no lifting kernel to carry the bias gradient: the
    // remap pass sums it while it copies (staged path: the separate passes of the reference)
    const bool fuse_bias_into_remap = bias_term && !fuse_bias_into_lift && !direct_weights && path_ >= PATH_FUSED;
    if (bias_term && !fuse_bias_into_lift && !direct_weights && !fuse_bias_into_remap) {
      begin(STAGE_BW_BIAS);
      DeviceMemoryPointer bias = p_bias_gradient_cube->get_device_pointer(p_driver);
      p_driver->backward_bias(&bias, &og, (int)(oR * oC), (int)oD, (int)iB);
      end(STAGE_BW_BIAS);
    }
    if (!direct_weights || strided_data) {
      begin(STAGE_BW_REMAP);
      p_forward_lower_connector->remap_output(*staging(), *output_g_cube, oB, num_output_features,
                                              fuse_bias_into_remap ? p_bias_gradient_cube : nullptr);
      end(STAGE_BW_REMAP);
    }
    LogicalCubeType lowered_outputgrad(direct_weights && !strided_data ? nullptr : staging()->get_p_data(),
                                       num_output_features, oR * oC * iB, 1, 1);
    if (needs_to_calc_backward_grad && !direct_data && !strided_direct_data) {
      begin(STAGE_GEMM_DATA);
      p_backward_gemm_updategrad_kernel->compute(&lowered_model, &lowered_outputgrad, backward_inputgrad());
      end(STAGE_GEMM_DATA);
    }
    // The weight-gradient GEMM is issued between the data-gradient GEMM and the lifting (the
    // reference runs it last, :619-621; the three results do not depend on each other): the
    // lifting kernel is HBM-bound and runs faster once the 1.8 GB written by the data-gradient
    // GEMM has drained from the caches.
    begin(STAGE_GEMM_WEIGHTS);
    if (direct_weights && strided_ok_) {
      p_driver->conv_strided_backward_weights(p_model_gradient_cube->get_p_data(),
                                              bias_term ? p_bias_gradient_cube->get_p_data() : nullptr,
                                              output_g_cube->get_p_data(), p_input_layer->p_data_cube->get_p_data(),
                                              (int)iB, (int)iD, (int)iR, (int)K, (int)stride, (int)padding,
                                              (int)num_output_features);
    } else if (direct_weights && small_kernels()) {
      p_driver->conv_small_backward_weights(p_model_gradient_cube->get_p_data(),
                                            bias_term ? p_bias_gradient_cube->get_p_data() : nullptr,
                                            output_g_cube->get_p_data(), p_input_layer->p_data_cube->get_p_data(),
                                            (int)iB, (int)iD, (int)iR, (int)K, (int)padding,
                                            (int)num_output_features);
    } else if (direct_weights) {
      p_driver->conv_direct_backward_weights(p_model_gradient_cube->get_p_data(),
                                             bias_term ? p_bias_gradient_cube->get_p_data() : nullptr,
                                             output_g_cube->get_p_data(), p_input_layer->p_data_cube->get_p_data(),
                                             (int)iB, (int)iD, (int)iR, (int)K, (int)padding,
                                             (int)num_output_features, in_image_stride_, out_image_stride_,
                                             (int)group);
    } else {
      p_backward_gemm_updateweight_kernel->alpha = 1.0;
      p_backward_gemm_updateweight_kernel->beta = 0.0;
      p_backward_gemm_updateweight_kernel->compute(&lowered_outputgrad, lowered(), &lowered_model_grad);
    }
    end(STAGE_GEMM_WEIGHTS);
    if (direct_data) {
      // remap + data-gradient GEMM + lifting in one kernel, reading the output gradient in place
      begin(STAGE_GEMM_DATA);
      p_driver->conv_direct_slabs(backward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                  (int)num_output_features, (int)iD, (int)K, 1, (int)group);
      p_driver->conv_direct_backward_data(input_g_cube->get_p_data(), output_g_cube->get_p_data(),
                                          backward_slabs()->get_p_data(), (int)iB, (int)iD, (int)iR, (int)K,
                                          (int)padding, (int)num_output_features, in_image_stride_,
                                          out_image_stride_,
                                          input_is_relu_output ? p_input_layer->p_data_cube->get_p_data() : nullptr,
                                          (int)group);
      end(STAGE_GEMM_DATA);
    } else if (strided_direct_data) {
      // remap + data-gradient GEMM + lifting of a strided layer in one kernel (phase decomposition)
      begin(STAGE_GEMM_DATA);
      p_driver->conv_strided_backward_data_slabs(backward_slabs()->get_p_data(), p_model_cube->get_p_data(),
                                                 (int)num_output_features, (int)iD, (int)K, (int)stride);
      p_driver->conv_strided_backward_data(input_g_cube->get_p_data(), output_g_cube->get_p_data(),
                                           backward_slabs()->get_p_data(), (int)iB, (int)iD, (int)iR, (int)K,
                                           (int)stride, (int)padding, (int)num_output_features);
      end(STAGE_GEMM_DATA);
      if (input_is_relu_output) {  // this kernel's store does not carry the mask
        DeviceMemoryPointer in_grad = input_g_cube->get_device_pointer(p_driver);
        p_driver->relu_backward(&in_grad, &in_grad, p_input_layer->p_data_cube->get_p_data());
      }
    } else if (needs_to_calc_backward_grad) {
      begin(STAGE_INVERSE_LOWER);
      if (fuse_bias_into_lift) {
        DeviceMemoryPointer input = input_g_cube->get_device_pointer(p_driver);
        DeviceMemoryPointer lowered_grad = backward_inputgrad()->get_device_pointer(p_driver);
        DeviceMemoryPointer bias = p_bias_gradient_cube->get_device_pointer(p_driver);
        p_driver->inverse_lower_cube_bias_backward(&input, &lowered_grad, p_forward_lower_connector->inverse_args(),
                                                   &bias, &og, (int)(oR * oC), (int)oD, (int)iB);
      } else {
        p_forward_lower_connector->inverse_lower_cube(backward_inputgrad(), input_g_cube);
      }
      end(STAGE_INVERSE_LOWER);
      if (input_is_relu_output) {  // the lowering path has no store to fold the mask into
        DeviceMemoryPointer in_grad = input_g_cube->get_device_pointer(p_driver);
        p_driver->relu_backward(&in_grad, &in_grad, p_input_layer->p_data_cube->get_p_data());
      }
    }
    report_backward_updateweight_history.end();
  }

 protected:
  LogicalCubeType *p_model_gradient_cube;
  LogicalCubeType *p_bias_gradient_cube;
  LogicalCubeType *p_forward_lowered_data;
  LogicalCubeType *p_backward_inputgrad;
  LogicalCubeType *p_staging_cube;
  LogicalCubeType *p_forward_slabs;   // model as zero-padded [d][o][k*k] for the direct forward kernel
  LogicalCubeType *p_backward_slabs;  // model as [o][d][k*k], filters reversed, for the direct data gradient
  Connector<DataType, DriverClass> *p_forward_lower_connector;
  Kernel<DataType, KernelConfig_GEMM_NOTRANS_TRANS_NO_DIM_FLIP, DriverClass> *p_forward_gemm_kernel;
  Kernel<DataType, KernelConfig_GEMM_NOTRANS_NOTRANS_DIM_FLIP, DriverClass> *p_backward_gemm_updateweight_kernel;
  Kernel<DataType, KernelConfig_GEMM_TRANS_NOTRANS, DriverClass> *p_backward_gemm_updategrad_kernel;

  // Fillers, src/bridges/ConvolutionBridge_impl.hxx:250-267.
  void initialize_logical_cube(const LogicalCubeType *cube, const cnn::FillerParameter &filler_param) {
    DeviceMemoryPointer data = cube->get_device_pointer(p_driver);
    const std::string &type = filler_param.type();
    if (type == "constant") {
      p_driver->sconstant_initialize(&data, (DataType)filler_param.value());
    } else if (type == "xavier") {
      p_driver->sinitialize_xavier(&data, cube->B, solver_param->random_seed());
    } else if (type == "bernoulli") {
      p_driver->sbernoulli_initialize(&data, (DataType)filler_param.value(), solver_param->random_seed());
    } else if (type == "gaussian") {
      p_driver->sgaussian_initialize(&data, (DataType)filler_param.mean(), (DataType)filler_param.std(),
                                     solver_param->random_seed());
    } else {
      host_fail("ERROR! INITIALIZATION TYPE NOT SUPPORTED: " + type);
    }
  }

 private:
  int path_ = PATH_FUSED, default_path_ = PATH_FUSED;
  size_t in_image_stride_ = 0, out_image_stride_ = 0;
  bool views_ = false;
  bool fuse_relu_ = false;
  bool direct_ok_ = false, strided_ok_ = false, strided_data_ok_ = false, profile_ = false;
  bool small_ok_ = false, use_small_ = true;
  bool pointwise_ok_ = false;  // 1 x 1, stride 1, no padding: products on the tensors as they lie
  LogicalCubeType *lowered() {
    if (!p_forward_lowered_data) p_forward_lowered_data = new LogicalCubeType(K * K * iD, oR * oC * iB, 1, 1, p_driver);
    return p_forward_lowered_data;
  }
  LogicalCubeType *backward_inputgrad() {
    if (!p_backward_inputgrad) p_backward_inputgrad = new LogicalCubeType(K * K * iD, oR * oC * iB, 1, 1, p_driver);
    return p_backward_inputgrad;
  }
  LogicalCubeType *staging() {  // [o][b][m*m] view of output / output gradient
    if (!p_staging_cube) p_staging_cube = new LogicalCubeType(oR, oC, oD, oB, p_driver);
    return p_staging_cube;
  }
  LogicalCubeType *forward_slabs() {
    if (!p_forward_slabs)
      p_forward_slabs = new LogicalCubeType(
          strided_ok_ ? p_driver->conv_strided_slab_floats((int)num_output_features, (int)iD, (int)K, (int)stride,
                                                           (int)padding)
                      : p_driver->conv_direct_slab_floats((int)num_output_features, (int)iD, (int)K, 0, (int)group),
          1, 1, 1, p_driver);
    return p_forward_slabs;
  }
  LogicalCubeType *backward_slabs() {
    if (!p_backward_slabs)
      p_backward_slabs = new LogicalCubeType(
          strided_data_ok_ ? p_driver->conv_strided_backward_data_slab_floats((int)num_output_features, (int)iD,
                                                                              (int)K, (int)stride)
                           : p_driver->conv_direct_slab_floats((int)num_output_features, (int)iD, (int)K, 1, (int)group),
          1, 1, 1, p_driver);
    return p_backward_slabs;
  }
  void *timers_[STAGE_COUNT];
  bool stage_ran_[STAGE_COUNT] = {};
  float stage_ms_[STAGE_COUNT];
  void begin(int s) {
    if (!profile_) return;
    if (!timers_[s]) cct_hip_timer_create(&timers_[s]);
    cct_hip_timer_start(timers_[s]);
  }
  void end(int s) {
    if (!profile_) return;
    cct_hip_timer_stop(timers_[s]);
    stage_ran_[s] = true;
    stage_kernel_[s] = cct_hip_last_kernel();
  }
  std::string stage_kernel_[STAGE_COUNT];
};

}  // namespace cct
