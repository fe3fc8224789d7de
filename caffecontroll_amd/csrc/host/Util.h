// Device-independent helpers (src/util.h:66-93).
#pragma once
#include <cassert>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "Fail.h"

namespace cct {

struct Util {
  // Learning-rate schedule of Util::get_learning_rate (src/util.h:76-93): the same policies and
  // the same float / double steps (pow and exp on float arguments are the float overloads, mixed
  // arguments promote to double, the result is rounded to float).  Returns false for a policy
  // the reference rejects ("multistep", unknown names) and leaves *rate untouched.
  static inline bool try_get_learning_rate(const std::string &lr_policy, float base_lr, float gamma, float iter,
                                           float caffe_stepsize, float power, float max_iter, float *rate) {
    if (lr_policy == "fixed") {
      *rate = base_lr;
    } else if (lr_policy == "step") {
      const float current_step = (float)(int)(iter / caffe_stepsize);
      *rate = base_lr * std::pow(gamma, current_step);
    } else if (lr_policy == "exp") {
      *rate = base_lr * std::pow(gamma, iter);
    } else if (lr_policy == "inv") {
      *rate = (float)(base_lr * std::pow(1.0 + gamma * iter, -power));
    } else if (lr_policy == "poly") {
      *rate = (float)(base_lr * std::pow(1.0 - (iter / max_iter), power));
    } else if (lr_policy == "sigmoid") {
      *rate = (float)(base_lr * (1.0 / (1.0 + std::exp(-gamma * (iter - caffe_stepsize)))));
    } else {
      return false;
    }
    return true;
  }

  // As above; an unknown policy ends the process, as the reference's assert does.
  static inline float get_learning_rate(const std::string &lr_policy, float base_lr, float gamma, float iter,
                                        float caffe_stepsize, float power, float max_iter) {
    float rate = 0.f;
    if (!try_get_learning_rate(lr_policy, base_lr, gamma, iter, caffe_stepsize, power, max_iter, &rate)) {
      host_fail("Unknown or unsupported learning rate policy: " + lr_policy);
    }
    return rate;
  }
};

}  // namespace cct
