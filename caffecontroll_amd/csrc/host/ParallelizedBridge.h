// Per-layer scheduler fixed at ONE device partition.
//
// Counterpart of ParallelizedBridge<DataType, BridgeType> (src/bridges/ParallelizedBridge.h,
// _impl.hxx:24-502, 508-753, 761-1141) in the configuration `gpu_0_batch_proportion: 1.0`:
// exactly one sub-bridge on the device that owns model, gradient and momentum
// (skip_model_copy_gpu, _impl.hxx:117), input/output layers shared with the neighbouring
// bridges in device memory, gradient update issued on the device (:993-995, :1057-1059).
// The reference's batch partitioning over CPU threads / several GPUs and the host gradient sum are
// not part of this build.
//
// Where the layers live (src/bridges/ParallelizedBridge.h:183-198, _impl.hxx:109-117, 217-267,
// 595-621, 686-705): by default the bridge shares device pointers with the bridges before and after
// it -- its input and output layers ARE device memory and nothing is copied, which is what
// DeepNet::construct_network arranges for consecutive device bridges.  With
// share_pointer_with_prev_bridge == false the input layer's cubes are HOST memory: the bridge owns
// device copies, uploads the input data at the start of forward() and downloads the input gradient
// at the end of backward().  With share_pointer_with_next_bridge == false the same holds for the
// output layer (data downloaded after forward(), gradient uploaded before backward()).  That is
// the mode the reference's own bridge tests run in (tests/test_parallelized_convolution.cpp).
// share_input_output_layer (ReLU, dropout: top == bottom) tells the bridge that its output layer
// is its input layer, so no output cubes exist.
//
// Where the reference issues one blocking copy before and one after the sub-bridge, a sub-bridge that
// can run on a range of images (ConvolutionBridge on its all-direct path) gets the batch in pieces
// through a staging pipe: piece i+1 uploads and piece i-1 downloads while piece i computes, the two
// directions of the link in use at once.  Every image's forward result and data gradient is independent
// of the other images, and the weight gradient is still ONE call over the whole batch once the last piece
// has arrived, so the results are those of the blocking sequence bit for bit (set_overlapped_staging(false)
// runs that sequence).  The overlap needs page-locked host cubes; with pageable ones the copies are
// correct but serialise.
#pragma once
#include "AbstractBridge.h"
#include "GradientUpdater.h"

namespace cct {

template <typename DataType, template <typename, typename> class BridgeType, typename DriverClass>
class ParallelizedBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  typedef Layer<DataType> LayerType;
  typedef LogicalCube<DataType> LogicalCubeType;
  typedef BridgeType<DataType, DriverClass> SubBridgeType;
  using Base::needs_to_calc_backward_grad;

  const size_t n_partition;  // always 1
  LogicalCubeType *p_model_cube;
  LogicalCubeType *p_model_grad;
  LogicalCubeType *p_bias_cube;
  LogicalCubeType *p_bias_grad;
  float model_base_learning_rate, bias_base_learning_rate;
  float model_base_regularization, bias_base_regularization;

  ParallelizedBridge(LayerType *const _input_layer, LayerType *const _output_layer,
                     const cnn::LayerParameter *const _layer_param, const cnn::SolverParameter *const _solver_param,
                     DriverClass *const _p_driver, size_t _n_partition = 1, size_t _n_thread_per_partition = 1,
                     bool _share_pointer_with_prev_bridge = true, bool _share_pointer_with_next_bridge = true,
                     bool _share_input_output_layer = false)
      : Base(_input_layer, _output_layer, _layer_param, _solver_param, _p_driver), n_partition(1),
        share_pointer_with_prev_bridge(_share_pointer_with_prev_bridge),
        share_pointer_with_next_bridge(_share_pointer_with_next_bridge),
        share_input_output_layer(_share_input_output_layer),
        p_model_cube(nullptr), p_model_grad(nullptr), p_bias_cube(nullptr), p_bias_grad(nullptr),
        model_base_learning_rate(_layer_param->blobs_lr(0)), bias_base_learning_rate(_layer_param->blobs_lr(1)),
        model_base_regularization(_layer_param->weight_decay(0)),
        bias_base_regularization(_layer_param->weight_decay(1)), p_grad_updater(nullptr),
        p_grad_updater_bias(nullptr) {
    (void)_n_thread_per_partition;
    if (_n_partition != 1 || _layer_param->gpu_0_batch_proportion() != 1.0f) {
      host_fail("ParallelizedBridge: this build runs one device partition (n_partition=1, gpu_0_batch_proportion=1.0)");
    }
    // device-side layers of the sub-bridge: the caller's own, or copies this bridge owns
    LayerType *sub_in = _input_layer, *sub_out = _output_layer;
    if (!share_pointer_with_prev_bridge) {
      p_device_input_layer = new LayerType(
          new LogicalCubeType(_input_layer->dR, _input_layer->dC, _input_layer->dD, _input_layer->dB, _p_driver),
          new LogicalCubeType(_input_layer->gR, _input_layer->gC, _input_layer->gD, _input_layer->gB, _p_driver));
      sub_in = p_device_input_layer;
    }
    if (share_input_output_layer) {
      sub_out = sub_in;
    } else if (!share_pointer_with_next_bridge) {
      p_device_output_layer = new LayerType(
          new LogicalCubeType(_output_layer->dR, _output_layer->dC, _output_layer->dD, _output_layer->dB, _p_driver),
          new LogicalCubeType(_output_layer->gR, _output_layer->gC, _output_layer->gD, _output_layer->gB, _p_driver));
      sub_out = p_device_output_layer;
    }
    p_sub_bridge = new SubBridgeType(sub_in, sub_out, _layer_param, _solver_param, _p_driver);
    p_model_cube = p_sub_bridge->get_model_cube();
    p_model_grad = p_sub_bridge->get_model_grad_cube();
    p_bias_cube = p_sub_bridge->get_bias_cube();
    p_bias_grad = p_sub_bridge->get_bias_grad_cube();
    if (p_model_cube)
      p_grad_updater = new SGDGradientUpdater<DataType, DriverClass>(
          (int)p_model_cube->n_elements, p_model_cube->get_p_data(), _solver_param, model_base_learning_rate,
          model_base_regularization, _p_driver);
    if (p_bias_cube)
      p_grad_updater_bias = new SGDGradientUpdater<DataType, DriverClass>(
          (int)p_bias_cube->n_elements, p_bias_cube->get_p_data(), _solver_param, bias_base_learning_rate,
          bias_base_regularization, _p_driver);
  }

  ~ParallelizedBridge() {
    if (pipe_) this->p_driver->pipe_destroy(pipe_);
    delete p_grad_updater;
    delete p_grad_updater_bias;
    delete p_sub_bridge;
    delete p_device_input_layer;
    delete p_device_output_layer;
  }

  // src/bridges/ParallelizedBridge.h:183-198 (the first and third are fixed at construction, as in
  // the reference; the second is set by the builder of the next bridge, src/DeepNet.h:1116-1120)
  bool get_share_pointer_with_prev_bridge() const { return share_pointer_with_prev_bridge; }
  bool get_share_pointer_with_next_bridge() const { return share_pointer_with_next_bridge; }
  bool get_share_input_output_layer() const { return share_input_output_layer; }
  // The builder of the next bridge raises the flag once it knows that bridge lives on the same device
  // (src/DeepNet.h:1116-1120): the output layer's cubes are then device memory the two bridges share.  The
  // device cubes this bridge allocated for a host-resident output become views of them (the sub-bridge keeps
  // its layer object) and the copies after forward() / before backward() stop.  Lowering the flag again would
  // need device cubes under a sub-bridge that was built on the caller's own layer: refused.
  void set_share_pointer_with_next_bridge(bool share) {
    if (share == share_pointer_with_next_bridge) return;
    if (!share || share_input_output_layer)
      host_fail("ParallelizedBridge: share_pointer_with_next_bridge can only be raised, and not on a bridge whose "
                "output layer is its input layer");
    if (p_device_output_layer) {
      p_device_output_layer->p_data_cube->adopt(this->p_output_layer->p_data_cube->get_p_data());
      p_device_output_layer->p_gradient_cube->adopt(this->p_output_layer->p_gradient_cube->get_p_data());
      output_is_view_ = true;
    }
    share_pointer_with_next_bridge = true;
  }

  SubBridgeType *sub_bridge() { return p_sub_bridge; }
  SGDGradientUpdater<DataType, DriverClass> *get_grad_updater() { return p_grad_updater; }
  SGDGradientUpdater<DataType, DriverClass> *get_grad_updater_bias() { return p_grad_updater_bias; }
  LogicalCubeType *get_model_cube() override { return p_model_cube; }
  LogicalCubeType *get_bias_cube() override { return p_bias_cube; }
  LogicalCubeType *get_model_grad_cube() override { return p_model_grad; }
  LogicalCubeType *get_bias_grad_cube() override { return p_bias_grad; }
  LogicalCubeType *get_model_history_cube() override {
    return p_grad_updater ? p_grad_updater->get_p_history_updates_cube() : nullptr;
  }
  LogicalCubeType *get_bias_history_cube() override {
    return p_grad_updater_bias ? p_grad_updater_bias->get_p_history_updates_cube() : nullptr;
  }
  // src/bridges/ParallelizedBridge.h:331-354: both updaters resume from `iter`
  void set_current_iter(int iter) override {
    if (p_grad_updater) p_grad_updater->set_current_iter(iter);
    if (p_grad_updater_bias) p_grad_updater_bias->set_current_iter(iter);
  }

  int get_current_iter() override {
    return p_grad_updater ? p_grad_updater->current_iter : p_grad_updater_bias ? p_grad_updater_bias->current_iter : -1;
  }

  // pieces the batch moves in when the layers are host resident and the sub-bridge can run on ranges
  // (false: the reference's blocking copy - compute - copy sequence)
  void set_overlapped_staging(bool on) { overlapped_ = on; }
  bool overlapped_staging() const { return overlapped_ && staged_ranges<SubBridgeType>(nullptr); }

  void forward() override {
    this->report_forward_history.reset();
    if ((p_device_input_layer || staged_output()) && overlapped_ && forward_in_pieces<SubBridgeType>(nullptr)) {
      this->report_forward_history.end();
      return;
    }
    if (p_device_input_layer) copy_cube(p_device_input_layer->p_data_cube, this->p_input_layer->p_data_cube, true);
    p_sub_bridge->forward();
    if (staged_output()) copy_cube(this->p_output_layer->p_data_cube, p_device_output_layer->p_data_cube, false);
    this->report_forward_history.end();
  }

  // sub-bridge backward, then the model and bias updates on the device
  void backward() override {
    this->report_backward_updateweight_history.reset();
    p_sub_bridge->needs_to_calc_backward_grad = needs_to_calc_backward_grad;
    if (!((p_device_input_layer || staged_output()) && overlapped_ && backward_in_pieces<SubBridgeType>(nullptr))) {
      if (staged_output())
        copy_cube(p_device_output_layer->p_gradient_cube, this->p_output_layer->p_gradient_cube, true);
      p_sub_bridge->backward();
      if (p_device_input_layer && needs_to_calc_backward_grad)
        copy_cube(this->p_input_layer->p_gradient_cube, p_device_input_layer->p_gradient_cube, false);
    }
    if (p_grad_updater) p_grad_updater->update(p_model_grad->get_p_data());
    if (p_grad_updater_bias) p_grad_updater_bias->update(p_bias_grad->get_p_data());
    this->report_backward_updateweight_history.end();
  }

 private:
  bool share_pointer_with_prev_bridge, share_pointer_with_next_bridge, share_input_output_layer;
  LayerType *p_device_input_layer = nullptr, *p_device_output_layer = nullptr;
  bool overlapped_ = true, output_is_view_ = false;
  cct_hip_pipe *pipe_ = nullptr;
  // the device copy of a host-resident output layer (null once the output is shared with the next bridge)
  LayerType *staged_output() const { return output_is_view_ ? nullptr : p_device_output_layer; }
  static constexpr size_t kPieces = 4;

  // Sub-bridges with forward_range / backward_data_range members take the batch in pieces; for every other
  // bridge type these overloads are chosen and report "not done" (SFINAE on the member's presence).
  template <typename S>
  bool staged_ranges(decltype(&S::forward_range)) const { return p_sub_bridge->supports_batch_ranges(); }
  template <typename S>
  bool staged_ranges(...) const { return false; }

  template <typename S>
  bool forward_in_pieces(decltype(&S::forward_range)) {
    S *sb = p_sub_bridge;
    if (!sb->supports_batch_ranges()) return false;
    if (!pipe_) pipe_ = this->p_driver->pipe_create();
    const size_t B = this->iB, pieces = B < kPieces ? B : kPieces;
    LogicalCubeType *h_in = this->p_input_layer->p_data_cube, *h_out = this->p_output_layer->p_data_cube;
    const size_t in_img = h_in->n_elements / B, out_img = h_out->n_elements / B;
    float *d_in = p_device_input_layer ? p_device_input_layer->p_data_cube->get_p_data() : nullptr;
    float *d_out = staged_output() ? p_device_output_layer->p_data_cube->get_p_data() : nullptr;
    int tickets[kPieces];
    this->p_driver->pipe_begin(pipe_);
    for (size_t i = 0; i < pieces; ++i) {
      const size_t b0 = i * B / pieces, b1 = (i + 1) * B / pieces;
      tickets[i] = d_in ? this->p_driver->pipe_upload(pipe_, d_in + b0 * in_img, h_in->get_p_data() + b0 * in_img,
                                                      (b1 - b0) * in_img * sizeof(DataType))
                        : -1;
    }
    sb->forward_prepare();
    for (size_t i = 0; i < pieces; ++i) {
      const size_t b0 = i * B / pieces, b1 = (i + 1) * B / pieces;
      if (tickets[i] >= 0) this->p_driver->pipe_wait_upload(pipe_, tickets[i]);
      sb->forward_range(b0, b1 - b0);
      if (d_out)
        this->p_driver->pipe_download(pipe_, h_out->get_p_data() + b0 * out_img, d_out + b0 * out_img,
                                      (b1 - b0) * out_img * sizeof(DataType));
    }
    this->p_driver->pipe_finish(pipe_);
    return true;
  }
  template <typename S>
  bool forward_in_pieces(...) { return false; }

  template <typename S>
  bool backward_in_pieces(decltype(&S::backward_data_range)) {
    S *sb = p_sub_bridge;
    if (!sb->supports_batch_ranges() || (needs_to_calc_backward_grad && !sb->backward_data_ranges_supported())) return false;
    if (!pipe_) pipe_ = this->p_driver->pipe_create();
    const size_t B = this->iB, pieces = B < kPieces ? B : kPieces;
    LogicalCubeType *h_ig = this->p_input_layer->p_gradient_cube, *h_og = this->p_output_layer->p_gradient_cube;
    const size_t in_img = this->p_input_layer->p_data_cube->n_elements / B, out_img = h_og->n_elements / B;
    float *d_ig = p_device_input_layer ? p_device_input_layer->p_gradient_cube->get_p_data() : nullptr;
    float *d_og = staged_output() ? p_device_output_layer->p_gradient_cube->get_p_data() : nullptr;
    int tickets[kPieces];
    this->p_driver->pipe_begin(pipe_);
    for (size_t i = 0; i < pieces; ++i) {
      const size_t b0 = i * B / pieces, b1 = (i + 1) * B / pieces;
      tickets[i] = d_og ? this->p_driver->pipe_upload(pipe_, d_og + b0 * out_img, h_og->get_p_data() + b0 * out_img,
                                                      (b1 - b0) * out_img * sizeof(DataType))
                        : -1;
    }
    if (needs_to_calc_backward_grad) {
      sb->backward_data_prepare();
      for (size_t i = 0; i < pieces; ++i) {
        const size_t b0 = i * B / pieces, b1 = (i + 1) * B / pieces;
        if (tickets[i] >= 0) this->p_driver->pipe_wait_upload(pipe_, tickets[i]);
        sb->backward_data_range(b0, b1 - b0);
        if (d_ig)
          this->p_driver->pipe_download(pipe_, h_ig->get_p_data() + b0 * in_img, d_ig + b0 * in_img,
                                        (b1 - b0) * in_img * sizeof(DataType));
      }
    } else {
      for (size_t i = 0; i < pieces; ++i)
        if (tickets[i] >= 0) this->p_driver->pipe_wait_upload(pipe_, tickets[i]);
    }
    // the whole output gradient is on the device by now: the weight (and bias) gradient in one call, as unpieced
    sb->backward_weights_all();
    this->p_driver->pipe_finish(pipe_);
    return true;
  }
  template <typename S>
  bool backward_in_pieces(...) { return false; }

  // host <-> device copy of a whole cube (synchronous, like the reference's driver memcpy)
  void copy_cube(LogicalCubeType *dst, LogicalCubeType *src, bool to_device) {
    DeviceMemoryPointer d = to_device ? dst->get_device_pointer(this->p_driver)
                                      : DeviceMemoryPointer_Local_RAM(dst->get_p_data(), dst->n_elements * sizeof(DataType));
    DeviceMemoryPointer s_ = to_device ? DeviceMemoryPointer_Local_RAM(src->get_p_data(), src->n_elements * sizeof(DataType))
                                       : src->get_device_pointer(this->p_driver);
    this->p_driver->memcpy(&d, &s_);
  }
  SubBridgeType *p_sub_bridge;
  SGDGradientUpdater<DataType, DriverClass> *p_grad_updater;
  SGDGradientUpdater<DataType, DriverClass> *p_grad_updater_bias;
};

}  // namespace cct
