// Base of all bridges for the HIP driver.  The reference keeps three copies of AbstractBridge
// (generic / CPUDriver / GPUDriver, src/bridges/AbstractBridge.h:229-631) and the generic one
// aborts for unknown drivers (:146,168); this is the specialisation a HIPDriver needs: layers
// hold device-resident cubes, so no host<->device staging happens inside a bridge.
#pragma once
#include <chrono>
#include <cstddef>

#include "LogicalCube.h"
#include "Params.h"

namespace cct {

// Wall-clock report kept per bridge (src/Report.h:14-91, reduced to what the path uses).
struct Report {
  double elapsed_s = 0.0;
  long n_runs = 0;
  std::chrono::steady_clock::time_point t0;
  void reset() { t0 = std::chrono::steady_clock::now(); }
  void end() {
    elapsed_s += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    ++n_runs;
  }
};

template <typename DataType, typename DriverClass>
class AbstractBridge {
 public:
  typedef Layer<DataType> InputLayerType;
  typedef Layer<DataType> OutputLayerType;
  typedef LogicalCube<DataType> LogicalCubeType;

  const size_t iR, iC, iD, iB;
  const size_t oR, oC, oD, oB;
  bool needs_to_calc_backward_grad;
  int run_with_n_threads;  // kept for interface parity; unused on the device
  Report report_forward_history, report_backward_updateweight_history;

  InputLayerType *const p_input_layer;
  OutputLayerType *const p_output_layer;
  const cnn::LayerParameter *const layer_param;
  const cnn::SolverParameter *const solver_param;
  DriverClass *const p_driver;

  AbstractBridge(InputLayerType *const _p_input_layer, OutputLayerType *const _p_output_layer,
                 const cnn::LayerParameter *const _layer_param, const cnn::SolverParameter *const _solver_param,
                 DriverClass *const _p_driver)
      : iR(_p_input_layer->dR), iC(_p_input_layer->dC), iD(_p_input_layer->dD), iB(_p_input_layer->dB),
        oR(_p_output_layer->dR), oC(_p_output_layer->dC), oD(_p_output_layer->dD), oB(_p_output_layer->dB),
        needs_to_calc_backward_grad(true), run_with_n_threads(1), p_input_layer(_p_input_layer),
        p_output_layer(_p_output_layer), layer_param(_layer_param), solver_param(_solver_param),
        p_driver(_p_driver) {}
  virtual ~AbstractBridge() {}

  virtual void forward() = 0;
  virtual void backward() = 0;

  // bridges without a model return NULL, as the reference's defaults do
  virtual LogicalCubeType *get_model_cube() { return nullptr; }
  virtual LogicalCubeType *get_bias_cube() { return nullptr; }
  virtual LogicalCubeType *get_model_grad_cube() { return nullptr; }
  virtual LogicalCubeType *get_bias_grad_cube() { return nullptr; }
  // momentum buffers of the two updaters and their iteration counter (what the reference's
  // snapshots carry besides the model: src/DeepNet.h:268-330, 386-422)
  virtual LogicalCubeType *get_model_history_cube() { return nullptr; }
  virtual LogicalCubeType *get_bias_history_cube() { return nullptr; }
  virtual void set_current_iter(int) {}
  virtual int get_current_iter() { return -1; }  // -1: no updater
};

}  // namespace cct
