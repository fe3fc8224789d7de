// SGD with momentum on the device.  Counterpart of GradientUpdater / SGDGradientUpdater
// (src/algorithms/GradientUpdater.h:30-51, 60-193): the same recurrence
//   g += lambda * w   (L2)   |   g += lambda * sign(w)   (L1)
//   h  = stepsize * g + momentum * h
//   w -= h
// issued as one kernel instead of three BLAS-1 calls (same fp32 roundings per element).
#pragma once
#include "LogicalCube.h"
#include "Params.h"
#include "Util.h"

namespace cct {

template <class DataType, class DriverClass>
class SGDGradientUpdater {
 public:
  typedef LogicalCube<DataType> LogicalCubeType;
  int current_iter;
  const int n_elements;
  DataType *const p_model;
  const cnn::SolverParameter *const p_solver;
  float base_learning_rate;
  float base_regularization;
  DriverClass *const p_driver;
  const float momentum;

  SGDGradientUpdater(int _n_elements, DataType *_p_model, const cnn::SolverParameter *const _p_solver, float _blr,
                     float _br, DriverClass *const _p_driver)
      : current_iter(0), n_elements(_n_elements), p_model(_p_model), p_solver(_p_solver),
        base_learning_rate(_blr), base_regularization(_br), p_driver(_p_driver), momentum(_p_solver->momentum()) {
    p_history_updates_cube = new LogicalCubeType(n_elements, 1, 1, 1, p_driver);
    DeviceMemoryPointer h = p_history_updates_cube->get_device_pointer(p_driver);
    p_driver->sconstant_initialize(&h, DataType(0.));
  }
  ~SGDGradientUpdater() { delete p_history_updates_cube; }

  float get_stepsize() {
    return base_learning_rate * Util::get_learning_rate(p_solver->lr_policy(), p_solver->base_lr(),
                                                        p_solver->gamma(), (float)current_iter,
                                                        (float)p_solver->stepsize(), p_solver->power(),
                                                        (float)p_solver->max_iter());
  }
  float get_weight_decay() { return p_solver->weight_decay() * base_regularization; }
  void set_current_iter(int _current_iter) { current_iter = _current_iter; }
  float get_momentum() const { return momentum; }
  LogicalCubeType *get_p_history_updates_cube() { return p_history_updates_cube; }

  void update(DataType *const p_gradient) {
    ++current_iter;
    const float stepsize = get_stepsize();
    const float lambda = get_weight_decay();
    const bool l1 = p_solver->regularization_type() == "L1";
    p_driver->sgd_update((size_t)n_elements, p_model, p_gradient, p_history_updates_cube->get_p_data(), stepsize,
                         momentum, lambda, l1);
  }

 private:
  LogicalCubeType *p_history_updates_cube;
};

}  // namespace cct
