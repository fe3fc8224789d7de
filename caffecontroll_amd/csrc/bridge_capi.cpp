// C entry points over the C++ host layer (see include/cct_bridge.h).
#include <cmath>
#include <exception>
#include <memory>
#include <string>

#include "../../include/cct_bridge.h"
#include "cct_common.h"
#include "host/ConvolutionBridge.h"
#include "host/Network.h"
#include "host/ParallelizedBridge.h"

using namespace cct;

namespace {

void fill_solver(cnn::SolverParameter &s, const cct_solver_param *p) {
  if (!p) return;
  s.base_lr_ = p->base_lr; s.momentum_ = p->momentum; s.gamma_ = p->gamma; s.power_ = p->power;
  s.weight_decay_ = p->weight_decay; s.stepsize_ = p->stepsize; s.max_iter_ = p->max_iter;
  s.random_seed_ = p->random_seed;
  if (p->lr_policy) s.lr_policy_ = p->lr_policy;
  if (p->regularization_type) s.regularization_type_ = p->regularization_type;
}

// Runs `body` with the host layer's failures turned into exceptions (Fail.h) and returns what it returns, or
// the error code with the message in cct_hip_last_error() if it throws: no failure inside a bridge ends
// the caller's process or crosses the C boundary as an exception.
template <typename F>
int guarded(const char *what, F body) {
  ErrorsAsExceptions scope;
  try {
    return body();
  } catch (const std::exception &e) {
    return cct::set_error(CCT_HIP_EINVAL, "%s: %s", what, e.what());
  } catch (...) {
    return cct::set_error(CCT_HIP_EINVAL, "%s: unknown failure", what);
  }
}

}  // namespace

struct cct_conv_bridge {
  HIPDriver driver;
  cnn::LayerParameter layer_param;
  cnn::SolverParameter solver_param;
  Layer<float> *in_layer = nullptr, *out_layer = nullptr;
  ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *pbridge = nullptr;
  ~cct_conv_bridge() {
    delete pbridge;
    delete in_layer;
    delete out_layer;
  }
};

extern "C" {

int cct_conv_bridge_create(cct_conv_bridge **out, int b, int d, int n, const cct_conv_param *conv,
                           const cct_solver_param *solver, float *in_data, float *in_grad, float *out_data,
                           float *out_grad) {
  return cct_conv_bridge_create_shared(out, b, d, n, conv, solver, in_data, in_grad, out_data, out_grad, 1, 1);
}

int cct_conv_bridge_create_shared(cct_conv_bridge **out, int b, int d, int n, const cct_conv_param *conv,
                                  const cct_solver_param *solver, float *in_data, float *in_grad, float *out_data,
                                  float *out_grad, int share_pointer_with_prev_bridge,
                                  int share_pointer_with_next_bridge) {
  if (!out || !conv || b <= 0 || d <= 0 || n <= 0 || conv->kernel_size <= 0 || conv->stride <= 0 ||
      conv->num_output <= 0 || conv->pad < 0 || n + 2 * conv->pad < conv->kernel_size || !in_data || !out_data)
    return cct::set_error(CCT_HIP_EINVAL, "conv_bridge_create: bad geometry or null tensor");
  if ((!share_pointer_with_prev_bridge && !in_grad) || (!share_pointer_with_next_bridge && !out_grad))
    return cct::set_error(CCT_HIP_EINVAL, "conv_bridge_create: a host-resident layer needs both of its cubes");
  *out = nullptr;
  return guarded("conv_bridge_create", [&] {
    std::unique_ptr<cct_conv_bridge> h(new cct_conv_bridge);  // its destructor frees what was built if a step throws
    const int k = conv->kernel_size, s = conv->stride, p = conv->pad, o = conv->num_output;
    const int m = (n + 2 * p - k) / s + 1;
    cnn::ConvolutionParameter &cp = h->layer_param.convolution_param_;
    cp.num_output_ = o; cp.kernel_size_ = k; cp.stride_ = s; cp.pad_ = p; cp.bias_term_ = conv->bias_term != 0;
    h->layer_param.blobs_lr_[0] = conv->lr_mult_weights; h->layer_param.blobs_lr_[1] = conv->lr_mult_bias;
    h->layer_param.weight_decay_[0] = conv->decay_mult_weights; h->layer_param.weight_decay_[1] = conv->decay_mult_bias;
    fill_solver(h->solver_param, solver);
    h->in_layer = new Layer<float>(new LogicalCube<float>(in_data, n, n, d, b),
                                   new LogicalCube<float>(in_grad, n, n, d, b));
    h->out_layer = new Layer<float>(new LogicalCube<float>(out_data, m, m, o, b),
                                    new LogicalCube<float>(out_grad, m, m, o, b));
    h->pbridge = new ParallelizedBridge<float, ConvolutionBridge, HIPDriver>(
        h->in_layer, h->out_layer, &h->layer_param, &h->solver_param, &h->driver, 1, 1,
        share_pointer_with_prev_bridge != 0, share_pointer_with_next_bridge != 0, false);
    *out = h.release();
    return 0;
  });
}

int cct_conv_bridge_destroy(cct_conv_bridge *h) {
  delete h;
  return 0;
}

int cct_conv_bridge_set_options(cct_conv_bridge *h, int fused, int profile, int needs_backward_grad) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("conv_bridge_set_options", [&] {
    if (fused >= 0) h->pbridge->sub_bridge()->set_path(fused);
    h->pbridge->sub_bridge()->set_stage_profiling(profile != 0);
    h->pbridge->needs_to_calc_backward_grad = needs_backward_grad != 0;
    h->pbridge->sub_bridge()->needs_to_calc_backward_grad = needs_backward_grad != 0;
    return 0;
  });
}

int cct_conv_bridge_path(cct_conv_bridge *h) { return h ? h->pbridge->sub_bridge()->path() : -1; }

int cct_conv_bridge_set_staging(cct_conv_bridge *h, int overlapped) {
  if (!h) return CCT_HIP_EINVAL;
  h->pbridge->set_overlapped_staging(overlapped != 0);
  return 0;
}

int cct_conv_bridge_share_with_next(cct_conv_bridge *h, float *out_data_device, float *out_grad_device) {
  if (!h || !out_data_device || !out_grad_device) return CCT_HIP_EINVAL;
  return guarded("conv_bridge_share_with_next", [&] {
    // the output layer's cubes now name the device memory of the next bridge's input layer
    h->out_layer->p_data_cube->set_p_data(out_data_device);
    h->out_layer->p_gradient_cube->set_p_data(out_grad_device);
    h->pbridge->set_share_pointer_with_next_bridge(true);
    return 0;
  });
}

int cct_conv_bridge_staging(cct_conv_bridge *h) { return h && h->pbridge->overlapped_staging() ? 1 : 0; }

float *cct_conv_bridge_model(cct_conv_bridge *h) { return h->pbridge->p_model_cube->get_p_data(); }
float *cct_conv_bridge_bias(cct_conv_bridge *h) {
  return h->pbridge->p_bias_cube ? h->pbridge->p_bias_cube->get_p_data() : nullptr;
}
float *cct_conv_bridge_model_grad(cct_conv_bridge *h) { return h->pbridge->p_model_grad->get_p_data(); }
float *cct_conv_bridge_bias_grad(cct_conv_bridge *h) {
  return h->pbridge->p_bias_grad ? h->pbridge->p_bias_grad->get_p_data() : nullptr;
}
float *cct_conv_bridge_lowered(cct_conv_bridge *h) {
  float *p = nullptr;  // the lowered cube is allocated on first use: NULL (and the error text) if that fails
  guarded("conv_bridge_lowered", [&] {
    p = h->pbridge->sub_bridge()->get_lowered_cube()->get_p_data();
    return 0;
  });
  return p;
}
float *cct_conv_bridge_history(cct_conv_bridge *h) {
  return h->pbridge->get_grad_updater()->get_p_history_updates_cube()->get_p_data();
}

int cct_conv_bridge_forward(cct_conv_bridge *h) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("conv_bridge_forward", [&] {
    h->pbridge->forward();
    return 0;
  });
}

int cct_conv_bridge_backward(cct_conv_bridge *h, int with_update) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("conv_bridge_backward", [&] {
    if (with_update) {
      h->pbridge->backward();
    } else {
      h->pbridge->sub_bridge()->needs_to_calc_backward_grad = h->pbridge->needs_to_calc_backward_grad;
      h->pbridge->sub_bridge()->backward();
    }
    return 0;
  });
}

int cct_conv_bridge_stage_ms(cct_conv_bridge *h, float ms[CCT_CONV_STAGE_COUNT]) {
  if (!h || !ms) return CCT_HIP_EINVAL;
  static_assert(CCT_CONV_STAGE_COUNT == STAGE_COUNT, "stage tables out of sync");
  for (int i = 0; i < STAGE_COUNT; ++i) ms[i] = h->pbridge->sub_bridge()->stage_ms(i);
  return 0;
}

const char *cct_conv_bridge_stage_kernel(cct_conv_bridge *h, int stage) {
  if (!h || stage < 0 || stage >= STAGE_COUNT) return "";
  return h->pbridge->sub_bridge()->stage_kernel(stage).c_str();
}

struct cct_net {
  Network *net;
};

int cct_net_validate(int batch, int depth, int size, const cct_layer_spec *layers, int n_layers,
                     const cct_solver_param *solver) {
  const std::string why = Network::validate(batch, depth, size, layers, n_layers, solver);
  return why.empty() ? 0 : cct::set_error(CCT_HIP_EINVAL, "net: %s", why.c_str());
}

int cct_net_create(cct_net **out, int batch, int depth, int size, const cct_layer_spec *layers, int n_layers,
                   const cct_solver_param *solver) {
  if (!out) return cct::set_error(CCT_HIP_EINVAL, "net_create: null result pointer");
  *out = nullptr;
  int rc = cct_net_validate(batch, depth, size, layers, n_layers, solver);
  if (rc) return rc;
  return guarded("net_create", [&] {
    Network *net = new Network(batch, depth, size, layers, n_layers, solver);
    cct_net *h = new cct_net;
    h->net = net;
    *out = h;
    return 0;
  });
}

int cct_net_destroy(cct_net *h) {
  if (!h) return 0;
  delete h->net;
  delete h;
  return 0;
}

float *cct_net_input(cct_net *h) { return h->net->input(); }
float *cct_net_labels(cct_net *h) { return h->net->labels(); }
int cct_net_num_layers(cct_net *h) { return h->net->num_layers(); }

void *cct_net_tensor(cct_net *h, int layer, int group, int which, size_t *n) {
  if (n) *n = 0;
  if (!h || layer < 0 || layer >= h->net->num_layers()) return nullptr;
  Network::Node &nd = h->net->node(layer);
  LogicalCube<float> *c = nullptr;
  if (which == 4 || which == 5) {  // tensors of the layer itself, whatever bridges it has (CONCAT has none)
    c = which == 4 ? nd.out->p_data_cube : nd.in->p_gradient_cube;
    if (n) *n = c->n_elements;
    return c->get_p_data();
  }
  // a grouped convolution run by one bridge: `group` selects that group's slice of the layer's model,
  // bias, gradients and momentum buffers ([o][d/g][k][k] and [o]: the groups lie one after another)
  const int layer_groups = nd.spec.type == CCT_LAYER_CONV && nd.spec.group > 1 ? nd.spec.group : 1;
  const bool sliced = layer_groups > 1 && nd.bridges.size() == 1 && which != 6;
  if (group < 0 || group >= (sliced ? layer_groups : (int)nd.bridges.size())) return nullptr;
  Network::BridgeT *b = nd.bridges[sliced ? 0 : group];
  switch (which) {
    case 0: c = b->get_model_cube(); break;
    case 1: c = b->get_bias_cube(); break;
    case 2: c = b->get_model_grad_cube(); break;
    case 3: c = b->get_bias_grad_cube(); break;
    case 4: c = nd.out->p_data_cube; break;
    case 5: c = nd.in->p_gradient_cube; break;
    case 7: c = b->get_model_history_cube(); break;
    case 8: c = b->get_bias_history_cube(); break;
    case 6:
      if (nd.spec.type == CCT_LAYER_DROPOUT) {
        auto *m = static_cast<DropoutBridge<float, HIPDriver> *>(b)->get_mask_cube();
        if (n) *n = m->n_elements;
        return m->get_p_data();
      }
      if (nd.spec.type == CCT_LAYER_MAXPOOL) {
        auto *m = static_cast<MaxPoolingBridge<float, HIPDriver> *>(b)->get_max_index_cube();
        if (n) *n = m->n_elements;
        return m->get_p_data();
      }
      return nullptr;
    default: return nullptr;
  }
  if (!c) return nullptr;
  if (sliced) {
    const size_t per_group = c->n_elements / layer_groups;
    if (n) *n = per_group;
    return c->get_p_data() + (size_t)group * per_group;
  }
  if (n) *n = c->n_elements;
  return c->get_p_data();
}

int cct_net_set_train(cct_net *h, int train) {
  if (!h) return CCT_HIP_EINVAL;
  h->net->set_train(train != 0);
  return 0;
}

int cct_net_set_conv_path(cct_net *h, int level) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("net_set_conv_path", [&] {
    for (int i = 0; i < h->net->num_layers(); ++i) {
      Network::Node &nd = h->net->node(i);
      if (nd.spec.type != CCT_LAYER_CONV) continue;
      for (auto *b : nd.bridges) {
        auto *cb = static_cast<ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *>(b)->sub_bridge();
        if (level < 0) cb->set_fused(true);
        else cb->set_path(level);
      }
    }
    return 0;
  });
}

int cct_net_freeze_dropout_masks(cct_net *h, int freeze) {
  if (!h) return CCT_HIP_EINVAL;
  for (int i = 0; i < h->net->num_layers(); ++i) {
    Network::Node &nd = h->net->node(i);
    if (nd.spec.type == CCT_LAYER_DROPOUT)
      static_cast<DropoutBridge<float, HIPDriver> *>(nd.bridges[0])->generate_mask = (freeze == 0);
  }
  return 0;
}

int cct_net_forward(cct_net *h) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("net_forward", [&] {
    h->net->forward();
    return 0;
  });
}

int cct_net_backward(cct_net *h) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("net_backward", [&] {
    h->net->backward();
    return 0;
  });
}

int cct_net_loss(cct_net *h, float *loss_sum) {
  if (!h || !loss_sum) return CCT_HIP_EINVAL;
  return guarded("net_loss", [&] {
    *loss_sum = h->net->loss();
    return 0;
  });
}

int cct_net_set_profiling(cct_net *h, int on) {
  if (!h) return CCT_HIP_EINVAL;
  return guarded("net_set_profiling", [&] {
    h->net->set_profiling(on != 0);
    return 0;
  });
}

int cct_net_layer_ms(cct_net *h, int layer, float *forward_ms, float *backward_ms) {
  if (!h || layer < 0 || layer >= h->net->num_layers()) return CCT_HIP_EINVAL;
  if (forward_ms) *forward_ms = h->net->layer_ms(layer, false);
  if (backward_ms) *backward_ms = h->net->layer_ms(layer, true);
  return 0;
}

int cct_net_update_ms(cct_net *h, float *ms) {
  if (!h || !ms) return CCT_HIP_EINVAL;
  *ms = h->net->update_ms();
  return 0;
}

namespace {
ConvolutionBridge<float, HIPDriver> *conv_of(cct_net *h, int layer, int bridge) {
  if (!h || layer < 0 || layer >= h->net->num_layers()) return nullptr;
  Network::Node &nd = h->net->node(layer);
  if (nd.spec.type != CCT_LAYER_CONV || bridge < 0 || bridge >= (int)nd.bridges.size()) return nullptr;
  return static_cast<ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *>(nd.bridges[bridge])->sub_bridge();
}
}  // namespace

int cct_net_conv_bridges(cct_net *h, int layer) {
  if (!h || layer < 0 || layer >= h->net->num_layers()) return 0;
  Network::Node &nd = h->net->node(layer);
  return nd.spec.type == CCT_LAYER_CONV ? (int)nd.bridges.size() : 0;
}

int cct_net_conv_stage_ms(cct_net *h, int layer, int bridge, float ms[CCT_CONV_STAGE_COUNT]) {
  auto *cb = conv_of(h, layer, bridge);
  if (!cb || !ms) return CCT_HIP_EINVAL;
  for (int i = 0; i < STAGE_COUNT; ++i) ms[i] = cb->stage_ms(i);
  return 0;
}

const char *cct_net_conv_stage_kernel(cct_net *h, int layer, int bridge, int stage) {
  auto *cb = conv_of(h, layer, bridge);
  if (!cb || stage < 0 || stage >= STAGE_COUNT) return "";
  return cb->stage_kernel(stage).c_str();
}

namespace {
int io_result(cct_net *h, bool ok) {
  return ok ? 0 : cct::set_error(CCT_HIP_EINVAL, "%s", h->net->io_error().c_str());
}
}  // namespace

int cct_net_write_model(cct_net *h, const char *file) {
  if (!h || !file) return CCT_HIP_EINVAL;
  return guarded("net_write_model", [&] { return io_result(h, h->net->write_blobs(file, Network::BLOB_MODEL)); });
}

int cct_net_read_model(cct_net *h, const char *file) {
  if (!h || !file) return CCT_HIP_EINVAL;
  return guarded("net_read_model", [&] { return io_result(h, h->net->read_blobs(file, Network::BLOB_MODEL)); });
}

int cct_net_write_snapshot(cct_net *h, const char *base_filename, int iter) {
  if (!h || !base_filename || iter < 0) return CCT_HIP_EINVAL;
  return guarded("net_write_snapshot", [&] { return io_result(h, h->net->write_snapshot(base_filename, iter)); });
}

int cct_net_read_snapshot(cct_net *h, const char *stem, int *iter) {
  if (!h || !stem) return CCT_HIP_EINVAL;
  return guarded("net_read_snapshot", [&] { return io_result(h, h->net->read_snapshot(stem, iter)); });
}

int cct_net_set_iter(cct_net *h, int iter) {
  if (!h || iter < 0) return CCT_HIP_EINVAL;
  return guarded("net_set_iter", [&] {
    h->net->set_current_iter(iter);
    return 0;
  });
}

int cct_net_get_iter(cct_net *h) { return h ? h->net->current_iter() : -1; }

int cct_net_num_classes(cct_net *h) { return h ? h->net->num_classes() : 0; }

size_t cct_net_parameter_size(cct_net *h) { return h ? h->net->parameter_size() : 0; }

float cct_solver_learning_rate(const cct_solver_param *solver, int iter) {
  float rate = NAN;
  if (!solver || !solver->lr_policy) return rate;
  Util::try_get_learning_rate(solver->lr_policy, solver->base_lr, solver->gamma, (float)iter, (float)solver->stepsize,
                              solver->power, (float)solver->max_iter, &rate);
  return rate;
}

}  // extern "C"
