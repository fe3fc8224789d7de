// Elementwise, pooling and loss operators for the HIP driver.  Counterparts of
//   ReLUBridge         src/bridges/ReLUBridge_impl.hxx:33-100
//   MaxPoolingBridge   src/bridges/MaxPoolingBridge_impl.hxx:13-151
//   LRNBridge          src/bridges/LRNBridge_impl.hxx:13-180
//   DropoutBridge      src/bridges/DropoutBridge_impl.hxx:13-194
//   SoftmaxLossBridge  src/bridges/SoftmaxLossBridge_impl.hxx:13-143
// Each forward()/backward() is one kernel on device-resident layers.
#pragma once
#include <climits>
#include <cstdio>
#include <cstdlib>

#include "AbstractBridge.h"

namespace cct {

#define CCT_BRIDGE_USINGS                                                                    \
  using Base::iR; using Base::iC; using Base::iD; using Base::iB;                            \
  using Base::oR; using Base::oC; using Base::oD; using Base::oB;                            \
  using Base::layer_param; using Base::solver_param; using Base::p_driver;                   \
  using Base::p_input_layer; using Base::p_output_layer;                                     \
  typedef Layer<DataType> LayerType;                                                         \
  typedef LogicalCube<DataType> LogicalCubeType;

// ---- ReLU: y = max(x, 0); dx = dy * (x > 0).  Works in place (input layer == output layer), the
// arrangement the reference uses on the GPU (share_input_output_layer).
template <typename DataType, typename DriverClass>
class ReLUBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  CCT_BRIDGE_USINGS
  ReLUBridge(LayerType *const in, LayerType *const out, const cnn::LayerParameter *const lp,
             const cnn::SolverParameter *const sp, DriverClass *const drv)
      : Base(in, out, lp, sp, drv) {
    if (oR != iR || oC != iC || oD != iD || oB != iB) {
      host_fail("ReLUBridge: input and output shapes differ");
    }
  }
  // set when the producing bridge clamps at zero while it stores (in-place ReLU after a convolution)
  bool forward_done_by_producer = false;
  void forward() override {
    if (forward_done_by_producer) return;
    DeviceMemoryPointer input = p_input_layer->p_data_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_data_cube->get_device_pointer(p_driver);
    p_driver->relu_forward(&output, &input);
  }
  // With shared layers the data cube holds y = max(x,0) by now; (y > 0) == (x > 0), so the same
  // mask results, as in the reference (ReLUBridge_impl.hxx:80-88 passes the input data pointer).
  // set when the consuming bridge (max pooling after an in-place ReLU) masks the gradient it stores
  bool backward_done_by_consumer = false;
  void backward() override {
    if (backward_done_by_consumer) return;
    DeviceMemoryPointer in_grad = p_input_layer->p_gradient_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer out_grad = p_output_layer->p_gradient_cube->get_device_pointer(p_driver);
    p_driver->relu_backward(&in_grad, &out_grad, p_input_layer->p_data_cube->get_p_data());
  }
};

// ---- max pooling, no padding, floor output size (src/DeepNet.h:1374-1376)
template <typename DataType, typename DriverClass>
class MaxPoolingBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  CCT_BRIDGE_USINGS
  const size_t kernel_size, stride;
  MaxPoolingBridge(LayerType *const in, LayerType *const out, const cnn::LayerParameter *const lp,
                   const cnn::SolverParameter *const sp, DriverClass *const drv)
      : Base(in, out, lp, sp, drv), kernel_size(lp->pooling_param().kernel_size()),
        stride(lp->pooling_param().stride()) {
    const size_t ph = (iR - kernel_size) / stride + 1, pw = (iC - kernel_size) / stride + 1;
    if (oR != ph || oC != pw || oD != iD || oB != iB) {
      host_fail("MaxPoolingBridge: inconsistent layer shapes");
    }
    max_index = new LogicalCube<int>(oR, oC, iD, iB, p_driver);
  }
  ~MaxPoolingBridge() { delete max_index; }
  LogicalCube<int> *get_max_index_cube() { return max_index; }
  void forward() override {
    DeviceMemoryPointer input = p_input_layer->p_data_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_data_cube->get_device_pointer(p_driver);
    p_driver->maxpool_forward(&output, &input, args());
  }
  void backward() override {
    DeviceMemoryPointer input = p_input_layer->p_gradient_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_gradient_cube->get_device_pointer(p_driver);
    if (input_is_relu_output && output_keeps_signs)
      p_driver->maxpool_backward_relu_pooled(&output, &input, args(), p_output_layer->p_data_cube->get_p_data());
    else if (input_is_relu_output)
      p_driver->maxpool_backward_relu(&output, &input, args(), p_input_layer->p_data_cube->get_p_data());
    else
      p_driver->maxpool_backward(&output, &input, args());
  }
  // the input layer is the output of an in-place ReLU whose backward this bridge performs while it
  // stores the gradient (the ReLU bridge then skips its own)
  bool input_is_relu_output = false;
  // the output cube still holds the pooled values (or at least their signs) when backward() runs:
  // true unless a layer that follows rewrites it in place with something other than a ReLU.  The
  // mask of the folded ReLU backward is then taken from the (four times smaller) output tensor.
  bool output_keeps_signs = false;

 private:
  LogicalCube<int> *max_index;
  _pool_forward_arg_helper args() const {
    _pool_forward_arg_helper a;
    a.stride = (int)stride; a.kernel_size = (int)kernel_size;
    a.iR = (int)iR; a.iC = (int)iC; a.oR = (int)oR; a.oC = (int)oC; a.D = (int)iD; a.B = (int)iB;
    a.max_index = max_index->get_p_data();
    return a;
  }
};

// ---- across-channel LRN; denoms (= scale) kept from forward to backward
template <typename DataType, typename DriverClass>
class LRNBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  CCT_BRIDGE_USINGS
  const float alpha, beta;
  const size_t local_size;
  LRNBridge(LayerType *const in, LayerType *const out, const cnn::LayerParameter *const lp,
            const cnn::SolverParameter *const sp, DriverClass *const drv)
      : Base(in, out, lp, sp, drv), alpha(lp->lrn_param().alpha()), beta(lp->lrn_param().beta()),
        local_size(lp->lrn_param().local_size()) {
    if (oR != iR || oC != iC || oD != iD || oB != iB || local_size % 2 != 1 || alpha < 0 || beta < 0) {
      host_fail("LRNBridge: bad shapes or parameters");
    }
    denoms = new LogicalCubeType(iR, iC, iD, iB, p_driver);
  }
  ~LRNBridge() { delete denoms; }
  void forward() override {
    DeviceMemoryPointer input = p_input_layer->p_data_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_data_cube->get_device_pointer(p_driver);
    _lrn_forward_arg_helper a2;
    a2.iR = (int)iR; a2.iC = (int)iC; a2.iD = (int)iD; a2.iB = (int)iB;
    a2.local_size = (int)local_size; a2.norm_window = (int)local_size / 2;
    a2.denoms = (char *)denoms->get_p_data();
    _lrn_forward_normalize_arg_helper a3;
    a3.alpha_over_size = alpha / local_size; a3.beta = beta; a3.denoms = (char *)denoms->get_p_data();
    p_driver->lrn_forward(&input, &output, a2, a3);
  }
  void backward() override {
    DeviceMemoryPointer input = p_input_layer->p_gradient_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_gradient_cube->get_device_pointer(p_driver);
    _lrn_backward_arg_helper a;
    a.oR = (int)oR; a.oC = (int)oC; a.oD = (int)oD; a.oB = (int)oB;
    a.alpha_over_size = alpha / local_size; a.beta = beta;
    a.local_size = (int)local_size; a.norm_window = (int)local_size / 2;
    a.denoms = (char *)denoms->get_p_data();
    a.input_data = (char *)p_input_layer->p_data_cube->get_p_data();
    a.output_data = (char *)p_output_layer->p_data_cube->get_p_data();
    p_driver->lrn_backward(&input, &output, a);
  }

 private:
  LogicalCubeType *denoms;
};

// ---- dropout: uint32 mask regenerated every training forward, keep iff mask > UINT_MAX*ratio,
// scale 1/(1-ratio); same mask in backward.  Test phase: copy (or nothing when layers are shared).
template <typename DataType, typename DriverClass>
class DropoutBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  CCT_BRIDGE_USINGS
  const float dropout_ratio;
  bool train;
  DropoutBridge(LayerType *const in, LayerType *const out, const cnn::LayerParameter *const lp,
                const cnn::SolverParameter *const sp, DriverClass *const drv)
      : Base(in, out, lp, sp, drv), dropout_ratio(lp->dropout_param().dropout_ratio()), train(true) {
    if (oR != iR || oC != iC || oD != iD || oB != iB || !(dropout_ratio < 1.f) || dropout_ratio < 0.f) {
      host_fail("DropoutBridge: bad shapes or ratio");
    }
    scale = (float)(1. / (1. - dropout_ratio));
    uint_thres_ = static_cast<unsigned int>(UINT_MAX * dropout_ratio);
    mask_cube = new LogicalCube<unsigned int>(iR, iC, iD, iB, p_driver);
    p_driver->init_rng(sp->random_seed());
  }
  ~DropoutBridge() { delete mask_cube; }
  LogicalCube<unsigned int> *get_mask_cube() { return mask_cube; }
  // generate_mask = false keeps the mask cube as it is (used to inject a known mask)
  bool generate_mask = true;
  void forward() override {
    DeviceMemoryPointer input = p_input_layer->p_data_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_data_cube->get_device_pointer(p_driver);
    if (train) {
      if (generate_mask) p_driver->rand_uint_initialize(mask_cube->get_p_data(), (int)mask_cube->n_elements);
      p_driver->dropout_forward_train(&output, &input, mask_cube->get_p_data(), scale, uint_thres_);
    } else if (output.ptr != input.ptr) {
      p_driver->memcpy(&output, &input);
    }
  }
  void backward() override {
    DeviceMemoryPointer input = p_input_layer->p_gradient_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_layer->p_gradient_cube->get_device_pointer(p_driver);
    p_driver->dropout_forward_train(&input, &output, mask_cube->get_p_data(), scale, uint_thres_);
  }

 private:
  float scale;
  unsigned int uint_thres_;
  LogicalCube<unsigned int> *mask_cube;
};

// ---- softmax + multinomial logistic loss on the device (the reference runs this bridge on the
// CPU driver only, SoftmaxLossBridge_impl.hxx:72-80).  Labels: one float per image.
template <typename DataType, typename DriverClass>
class SoftmaxLossBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  CCT_BRIDGE_USINGS
  LogicalCubeType *const p_data_labels;  // [1][1][1][B], device
  SoftmaxLossBridge(LayerType *const in, LayerType *const out, const cnn::LayerParameter *const lp,
                    const cnn::SolverParameter *const sp, DriverClass *const drv,
                    LogicalCubeType *const _p_data_labels)
      : Base(in, out, lp, sp, drv), p_data_labels(_p_data_labels) {
    if (oR != iR || oC != iC || oD != iD || oB != iB || _p_data_labels->n_elements != iB) {
      host_fail("SoftmaxLossBridge: bad shapes");
    }
    loss_device = new LogicalCubeType(1, 1, 1, 1, p_driver);
  }
  ~SoftmaxLossBridge() { delete loss_device; }
  // Training: forward() also writes the input gradient (the launch that computes the probabilities holds
  // everything the gradient needs), and the backward() that follows it has nothing left to do.  Set by the
  // owner of the chain when every forward pass is followed by a backward pass; a backward() without a
  // forward() since the last one computes the gradient from the stored probabilities as usual.
  bool gradient_with_forward = false;
  // probabilities go to the output layer's data cube; the batch-summed loss stays on the device
  void forward() override {
    if (gradient_with_forward) {
      p_driver->softmax_loss_forward_backward(p_output_layer->p_data_cube->get_p_data(),
                                              p_input_layer->p_gradient_cube->get_p_data(),
                                              p_input_layer->p_data_cube->get_p_data(), p_data_labels->get_p_data(),
                                              loss_device->get_p_data(), (int)(iR * iC * iD), (int)iB, (int)(iR * iC));
      gradient_is_current_ = true;
      return;
    }
    p_driver->softmax_loss_forward(p_output_layer->p_data_cube->get_p_data(), p_input_layer->p_data_cube->get_p_data(),
                                   p_data_labels->get_p_data(), loss_device->get_p_data(), (int)(iR * iC * iD),
                                   (int)iB);
    gradient_is_current_ = false;
  }
  // input gradient = (prob - onehot) / B / (R*C), from the probabilities stored by forward()
  void backward() override {
    if (gradient_is_current_) {
      gradient_is_current_ = false;
      return;
    }
    p_driver->softmax_loss_backward(p_input_layer->p_gradient_cube->get_p_data(),
                                    p_output_layer->p_data_cube->get_p_data(), p_data_labels->get_p_data(),
                                    (int)(iR * iC * iD), (int)iB, (int)(iR * iC));
  }
  // summed loss over the batch (one synchronous 4-byte copy); callers divide by B (src/DeepNet.h:2139)
  float get_loss() {
    float v = 0.f;
    DeviceMemoryPointer_Local_RAM host(&v, sizeof(float));
    DeviceMemoryPointer dev = loss_device->get_device_pointer(p_driver);
    p_driver->memcpy(&host, &dev);
    return v;
  }

 private:
  LogicalCubeType *loss_device;
  bool gradient_is_current_ = false;
};

#undef CCT_BRIDGE_USINGS

}  // namespace cct
