// Per-layer scheduler fixed at ONE device partition.
//
// Counterpart of ParallelizedBridge<DataType, BridgeType> (src/bridges/ParallelizedBridge.h,
// _impl.hxx:24-502, 508-753, 761-1141) in the configuration `gpu_0_batch_proportion: 1.0`:
// exactly one sub-bridge on the device that owns model, gradient and momentum
// (skip_model_copy_gpu, _impl.hxx:117), input/output layers shared with the neighbouring
// bridges in device memory, gradient update issued on the device (:993-995, :1057-1059).
// The reference's batch partitioning over CPU threads / several GPUs, the host<->device copies
// and the host gradient sum are not part of this build.
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
                     DriverClass *const _p_driver, size_t _n_partition = 1, size_t _n_thread_per_partition = 1)
      : Base(_input_layer, _output_layer, _layer_param, _solver_param, _p_driver), n_partition(1),
        p_model_cube(nullptr), p_model_grad(nullptr), p_bias_cube(nullptr), p_bias_grad(nullptr),
        model_base_learning_rate(_layer_param->blobs_lr(0)), bias_base_learning_rate(_layer_param->blobs_lr(1)),
        model_base_regularization(_layer_param->weight_decay(0)),
        bias_base_regularization(_layer_param->weight_decay(1)), p_grad_updater(nullptr),
        p_grad_updater_bias(nullptr) {
    (void)_n_thread_per_partition;
    if (_n_partition != 1 || _layer_param->gpu_0_batch_proportion() != 1.0f) {
      std::fprintf(stderr, "ParallelizedBridge: this build runs one device partition "
                           "(n_partition=1, gpu_0_batch_proportion=1.0)\n");
      std::abort();
    }
    p_sub_bridge = new SubBridgeType(_input_layer, _output_layer, _layer_param, _solver_param, _p_driver);
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
    delete p_grad_updater;
    delete p_grad_updater_bias;
    delete p_sub_bridge;
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

  void forward() override {
    this->report_forward_history.reset();
    p_sub_bridge->forward();
    this->report_forward_history.end();
  }

  // sub-bridge backward, then the model and bias updates on the device
  void backward() override {
    this->report_backward_updateweight_history.reset();
    p_sub_bridge->needs_to_calc_backward_grad = needs_to_calc_backward_grad;
    p_sub_bridge->backward();
    if (p_grad_updater) p_grad_updater->update(p_model_grad->get_p_data());
    if (p_grad_updater_bias) p_grad_updater_bias->update(p_bias_grad->get_p_data());
    this->report_backward_updateweight_history.end();
  }

 private:
  SubBridgeType *p_sub_bridge;
  SGDGradientUpdater<DataType, DriverClass> *p_grad_updater;
  SGDGradientUpdater<DataType, DriverClass> *p_grad_updater_bias;
};

}  // namespace cct
