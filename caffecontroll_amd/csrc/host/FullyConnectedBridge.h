// Fully connected operator for the HIP driver: three sgemm_new calls, no lowering.
// Counterpart of FullyConnectedBridge (src/bridges/FullyConnectedBridge_impl.hxx:13-110 ctor,
// 169-234 forward, 255-326 backward).  The model cube is [oD][iD][K][K] with K = iR, i.e. the
// GEMM matrix [O x I] with I = iR*iC*iD.
#pragma once
#include <cstdio>
#include <cstdlib>

#include "AbstractBridge.h"

namespace cct {

template <typename DataType, typename DriverClass>
class FullyConnectedBridge : public AbstractBridge<DataType, DriverClass> {
  typedef AbstractBridge<DataType, DriverClass> Base;

 public:
  using Base::iR; using Base::iC; using Base::iD; using Base::iB;
  using Base::oR; using Base::oC; using Base::oD; using Base::oB;
  using Base::needs_to_calc_backward_grad;
  using Base::layer_param; using Base::solver_param; using Base::p_driver;
  using Base::p_input_layer; using Base::p_output_layer;
  typedef Layer<DataType> LayerType;
  typedef LogicalCube<DataType> LogicalCubeType;

  const size_t K;
  const size_t num_output_features;
  const bool bias_term;
  LogicalCubeType *p_model_cube;
  LogicalCubeType *p_bias_cube;

  FullyConnectedBridge(LayerType *const _p_input_layer, LayerType *const _p_output_layer,
                       const cnn::LayerParameter *const _layer_param,
                       const cnn::SolverParameter *const _solver_param, DriverClass *const _p_driver)
      : Base(_p_input_layer, _p_output_layer, _layer_param, _solver_param, _p_driver), K(_p_input_layer->dR),
        num_output_features(_layer_param->inner_product_param().num_output()),
        bias_term(_layer_param->inner_product_param().bias_term()), p_model_cube(nullptr), p_bias_cube(nullptr),
        p_bias_gradient_cube(nullptr) {
    if (oR != 1 || oC != 1 || iB != oB || oD != num_output_features || iR != iC) {
      host_fail("FullyConnectedBridge: inconsistent layer shapes");
    }
    p_model_cube = new LogicalCubeType(K, K, iD, oD, p_driver);
    initialize_logical_cube(p_model_cube, _layer_param->inner_product_param().weight_filler());
    p_model_gradient_cube = new LogicalCubeType(K, K, iD, oD, p_driver);
    DeviceMemoryPointer mg = p_model_gradient_cube->get_device_pointer(p_driver);
    p_driver->sconstant_initialize(&mg, DataType(0.));
    if (bias_term) {
      p_bias_cube = new LogicalCubeType(1, 1, oD, 1, p_driver);
      initialize_logical_cube(p_bias_cube, _layer_param->inner_product_param().bias_filler());
      p_bias_gradient_cube = new LogicalCubeType(1, 1, oD, 1, p_driver);
      DeviceMemoryPointer bg = p_bias_gradient_cube->get_device_pointer(p_driver);
      p_driver->sconstant_initialize(&bg, DataType(0.));
    }
    // GEMM dimensions, named as in the reference
    data_R = (int)iB;                 // rows of the data matrix (batch)
    data_C = (int)(iR * iC * iD);     // its columns (features in)
    model_R = (int)oD;                // rows of the model matrix (features out)
    model_C = data_C;
    // a handful of outputs: one launch per pass instead of GEMM + split-K reduction + bias passes
    small_ = p_driver->fc_small_supported(data_R, data_C, model_R);
  }

  ~FullyConnectedBridge() {
    delete p_model_cube;
    delete p_model_gradient_cube;
    delete p_bias_cube;
    delete p_bias_gradient_cube;
  }

  LogicalCubeType *get_model_cube() override { return p_model_cube; }
  LogicalCubeType *get_bias_cube() override { return p_bias_cube; }
  LogicalCubeType *get_model_grad_cube() override { return p_model_gradient_cube; }
  LogicalCubeType *get_bias_grad_cube() override { return p_bias_gradient_cube; }

  // Y[B x O] = X[B x I] * W^T + bias: the reference's non-CPU branch runs sgemm_new and then
  // forward_bias with a 1x1 feature map (:224-228); here the bias, and the clamp of an in-place ReLU
  // that directly follows (set_fuse_relu), ride on the GEMM's output pass -- the same sums in the
  // same order, two or three launches fewer per layer.
  void set_fuse_relu(bool on) { fuse_relu_ = on; }
  // The input layer is the output of an in-place ReLU whose backward this bridge performs on the input
  // gradient it produces (the ReLU bridge then skips its own): masked in the store of the small-layer
  // kernel, else by a pass after the data-gradient GEMM.  Only meaningful with needs_to_calc_backward_grad.
  bool input_is_relu_output = false;
  // false: always the three GEMMs (what tests compare the one-launch kernels with)
  void set_small_kernels(bool on) { small_ = on && p_driver->fc_small_supported(data_R, data_C, model_R); }
  bool small_kernels() const { return small_; }
  void forward() override {
    this->report_forward_history.reset();
    LogicalCubeType *input_d_cube = p_input_layer->p_data_cube;
    LogicalCubeType *output_d_cube = p_output_layer->p_data_cube;
    if (small_) {
      p_driver->fc_small_forward(output_d_cube->get_p_data(), input_d_cube->get_p_data(), p_model_cube->get_p_data(),
                                 bias_term ? p_bias_cube->get_p_data() : nullptr, data_R, data_C, model_R, fuse_relu_);
      this->report_forward_history.end();
      return;
    }
    p_driver->sgemm_new_bias(CblasNoTrans, CblasTrans, data_R, model_R, model_C, 1.f, input_d_cube->get_p_data(),
                             p_model_cube->get_p_data(), 0.f, output_d_cube->get_p_data(),
                             bias_term ? p_bias_cube->get_p_data() : nullptr, fuse_relu_);
    this->report_forward_history.end();
  }

  // db = dY^T * ones;  dX[B x I] = dY * W;  dW[O x I] = dY^T * X
  void backward() override {
    this->report_backward_updateweight_history.reset();
    LogicalCubeType *output_g_cube = p_output_layer->p_gradient_cube;
    LogicalCubeType *input_g_cube = p_input_layer->p_gradient_cube;
    LogicalCubeType *input_d_cube = p_input_layer->p_data_cube;
    if (small_) {
      p_driver->fc_small_backward(needs_to_calc_backward_grad ? input_g_cube->get_p_data() : nullptr,
                                  p_model_gradient_cube->get_p_data(),
                                  bias_term ? p_bias_gradient_cube->get_p_data() : nullptr, output_g_cube->get_p_data(),
                                  input_d_cube->get_p_data(), p_model_cube->get_p_data(), data_R, data_C, model_R,
                                  needs_to_calc_backward_grad && input_is_relu_output ? input_d_cube->get_p_data()
                                                                                      : nullptr);
      this->report_backward_updateweight_history.end();
      return;
    }
    if (bias_term && !needs_to_calc_backward_grad) {
      DeviceMemoryPointer output = output_g_cube->get_device_pointer(p_driver);
      DeviceMemoryPointer bias = p_bias_gradient_cube->get_device_pointer(p_driver);
      p_driver->backward_bias_fc(&bias, &output, (int)oD, (int)iB);
    }
    // the reference always computes the data gradient here (:306-308); it is skipped when the
    // caller says the layer below does not need it.  The bias gradient (the same bits as backward_bias_fc's) goes
    // with it: both read the output gradient, and the product's reduction launch has workgroups to spare.
    if (needs_to_calc_backward_grad) {
      p_driver->sgemm_new_colsum(CblasNoTrans, CblasNoTrans, data_R, model_C, model_R, 1.f, output_g_cube->get_p_data(),
                                 p_model_cube->get_p_data(), 0.f, input_g_cube->get_p_data(),
                                 bias_term ? p_bias_gradient_cube->get_p_data() : nullptr, output_g_cube->get_p_data(),
                                 bias_term ? (int)iB : 0, bias_term ? (int)oD : 0);
      if (input_is_relu_output) {  // the GEMM has no store to fold the mask into
        DeviceMemoryPointer in_grad = input_g_cube->get_device_pointer(p_driver);
        p_driver->relu_backward(&in_grad, &in_grad, input_d_cube->get_p_data());
      }
    }
    p_driver->sgemm_new(CblasTrans, CblasNoTrans, model_R, model_C, data_R, 1.f, output_g_cube->get_p_data(),
                        input_d_cube->get_p_data(), 0.f, p_model_gradient_cube->get_p_data());
    this->report_backward_updateweight_history.end();
  }

 protected:
  LogicalCubeType *p_model_gradient_cube;
  LogicalCubeType *p_bias_gradient_cube;
  int data_R, data_C, model_R, model_C;
  bool fuse_relu_ = false, small_ = false;

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
};

}  // namespace cct
