// Bridges on the HIP driver, each wrapped in a one-partition ParallelizedBridge: the device-resident
// equivalent of what DeepNet::construct_network builds from a prototxt (src/DeepNet.h:968-2030) and
// of run_forward_pass / run_backward_pass (src/DeepNet.h:171-266).  Layer descriptions come as a C
// array instead of a parsed prototxt, in the prototxt's order; each layer reads the one before it
// (LeNet, CaffeNet) or the layers its `bottoms` name (the reference's two-tower networks).
//
// Graph rules (src/DeepNet.h:1700-1757, 1924-2028):
//   * a layer output read by several layers is shared, not copied: every reader sees the same data
//     cube; the first reader writes its gradient into the producer's gradient cube, every further
//     reader into a cube of its own, and before the producer's (or the last in-place layer's)
//     backward step the extra cubes are added to the first in reader order -- the sum the
//     reference's Split bridge forms;
//   * CONCAT stacks its bottoms along the depth: forward copies each bottom into its channel slice
//     of the output, backward copies the slices of the output gradient back;
//   * a layer computes an input gradient only if some layer with weights lies upstream of it.
//
// Placement rules kept from the reference:
//   * output sizes: conv (R+2p-K)/s+1 (:112-115), pooling floor((R-K)/s)+1 unpadded (:1374-1376);
//   * the first weight layer does not compute a data gradient (:1108-1110);
//   * ReLU and dropout run in place on their input layer (the reference shares the layers on the
//     GPU: ParallelizedBridge.h:183-198); an in-place ReLU directly after a convolution is applied
//     by the convolution's output store (same values, one pass over the tensor less);
//   * `group` > 1 is `group` independent convolutions on channel slices whose outputs are
//     concatenated along depth (the reference's two-tower Split/Concat arrangement,
//     src/DeepNet.h:1700-1757): one bridge that runs all groups in each of its launches when the
//     direct kernels take the layer, otherwise one bridge per group on contiguous copies of the
//     slices, moved with a strided device copy.
//
// Model files and snapshots use the reference's format (src/DeepNet.h:268-422): raw fp32, for
// every bridge in order its model cube and then its bias cube; a snapshot is three files
// <base>.snapshot_iter<N>.{MODEL,HISTORY,ITER}.bin (weights, momentum buffers, one int).
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/cct_bridge.h"
#include "ConvolutionBridge.h"
#include "FullyConnectedBridge.h"
#include "ParallelizedBridge.h"
#include "SimpleBridges.h"

namespace cct {

class Network {
 public:
  typedef Layer<float> LayerT;
  typedef LogicalCube<float> CubeT;
  typedef AbstractBridge<float, HIPDriver> BridgeT;

  struct Node {
    cct_layer_spec spec;
    LayerT *in = nullptr;   // the (first) bottom as this node sees it; not owned here (owned through layers_)
    LayerT *out = nullptr;
    std::vector<LayerT *> ins;                   // every bottom (CONCAT has several)
    bool run_backward = true;                    // false: no layer with weights upstream and none here
    std::vector<BridgeT *> bridges;              // 1; one per group for a grouped conv off the direct kernels
    std::vector<LayerT *> group_in, group_out;   // per-group contiguous layers (grouped conv only)
    std::vector<cnn::LayerParameter *> params;
  };

  // What the filler draws (cct_hip_fill_*) would refuse, said before anything is built; NULL if fine.
  static const char *bad_filler(const cct_filler &f) {
    if (f.type < 0 || f.type > 3) return "unknown filler type";
    if (f.type == CCT_FILLER_GAUSSIAN && !(f.std >= 0.f && std::isfinite(f.std) && std::isfinite(f.mean)))
      return "gaussian std must be finite and not negative";
    if (f.type == CCT_FILLER_BERNOULLI && !(f.value >= 0.f && f.value <= 1.f))
      return "bernoulli probability must be in [0, 1]";
    if (f.type == CCT_FILLER_CONSTANT && !std::isfinite(f.value)) return "constant value must be finite";
    return nullptr;
  }

  // Walks the chain with the reference's size rules (conv (R+2p-K)/s+1, src/DeepNet.h:112-115;
  // pooling (R-K)/s+1, :1374-1376) and returns "" if every layer can be built, else a message that
  // names the layer.  Host arithmetic only; the constructor runs it first, so a bad description
  // ends in an exception instead of an unsigned wrap-around, a division by zero or a huge allocation.
  static std::string validate(int batch, int depth, int size, const cct_layer_spec *specs, int n_specs,
                              const cct_solver_param *sp) {
    auto at = [](int i, const std::string &what) { return "layer " + std::to_string(i) + ": " + what; };
    if (batch <= 0 || depth <= 0 || size <= 0) return "batch, depth and size must be positive";
    if (!specs || n_specs <= 0) return "no layers";
    if (sp) {
      float r;
      if (sp->lr_policy && !Util::try_get_learning_rate(sp->lr_policy, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, &r))
        return std::string("unknown or unsupported lr_policy \"") + sp->lr_policy + "\"";
      if (sp->lr_policy && std::string(sp->lr_policy) == "step" && sp->stepsize <= 0)
        return "lr_policy \"step\" needs stepsize >= 1";
      if (sp->lr_policy && std::string(sp->lr_policy) == "poly" && sp->max_iter <= 0)
        return "lr_policy \"poly\" needs max_iter >= 1";
      if (sp->regularization_type && std::string(sp->regularization_type) != "L2" &&
          std::string(sp->regularization_type) != "L1")
        return std::string("regularization_type must be L2 or L1, not \"") + sp->regularization_type + "\"";
    }
    std::vector<long> Rs(n_specs), Ds(n_specs);
    for (int i = 0; i < n_specs; ++i) {
      const cct_layer_spec &s = specs[i];
      if (s.n_bottoms < 0 || s.n_bottoms > CCT_MAX_BOTTOMS) return at(i, "n_bottoms out of range");
      if (s.type != CCT_LAYER_CONCAT && s.n_bottoms > 1) return at(i, "only CONCAT reads more than one layer");
      if (s.type == CCT_LAYER_CONCAT && s.n_bottoms < 2) return at(i, "CONCAT needs at least two bottoms");
      for (int j = 0; j < s.n_bottoms; ++j)
        if (s.bottoms[j] < -1 || s.bottoms[j] >= i)
          return at(i, "bottom " + std::to_string(s.bottoms[j]) + " is not the network input (-1) or an earlier layer");
      const int b0 = s.n_bottoms ? s.bottoms[0] : i - 1;
      long R = b0 < 0 ? size : Rs[b0], D = b0 < 0 ? depth : Ds[b0];
      switch (s.type) {
        case CCT_LAYER_CONV: {
          if (s.num_output <= 0) return at(i, "convolution needs num_output >= 1");
          if (s.kernel_size < 1 || s.stride < 1 || s.pad < 0)
            return at(i, "convolution needs kernel_size >= 1, stride >= 1 and pad >= 0");
          if (s.kernel_size > R + 2L * s.pad)
            return at(i, "kernel_size " + std::to_string(s.kernel_size) + " exceeds the padded input (" +
                             std::to_string(R + 2L * s.pad) + ")");
          const int g = s.group > 1 ? s.group : 1;
          if (D % g || s.num_output % g) return at(i, "group must divide input depth and num_output");
          if (const char *why = bad_filler(s.weight_filler)) return at(i, std::string("weight filler: ") + why);
          if (const char *why = bad_filler(s.bias_filler)) return at(i, std::string("bias filler: ") + why);
          R = (R + 2L * s.pad - s.kernel_size) / s.stride + 1;
          D = s.num_output;
          break;
        }
        case CCT_LAYER_FC:
          if (s.num_output <= 0) return at(i, "inner product needs num_output >= 1");
          if (const char *why = bad_filler(s.weight_filler)) return at(i, std::string("weight filler: ") + why);
          if (const char *why = bad_filler(s.bias_filler)) return at(i, std::string("bias filler: ") + why);
          R = 1;
          D = s.num_output;
          break;
        case CCT_LAYER_MAXPOOL:
          if (s.kernel_size < 1 || s.stride < 1) return at(i, "pooling needs kernel_size >= 1 and stride >= 1");
          if (s.kernel_size > R)
            return at(i, "pooling kernel_size " + std::to_string(s.kernel_size) + " exceeds the input (" +
                             std::to_string(R) + ")");
          R = (R - s.kernel_size) / s.stride + 1;
          break;
        case CCT_LAYER_LRN:
          if (s.lrn_local_size < 1 || s.lrn_local_size % 2 == 0) return at(i, "LRN local_size must be odd and >= 1");
          if (!std::isfinite(s.lrn_alpha) || !std::isfinite(s.lrn_beta)) return at(i, "LRN alpha and beta must be finite");
          break;
        case CCT_LAYER_DROPOUT:
          if (!(s.dropout_ratio >= 0.f && s.dropout_ratio < 1.f)) return at(i, "dropout_ratio must be in [0, 1)");
          break;
        case CCT_LAYER_CONCAT:
          D = 0;
          for (int j = 0; j < s.n_bottoms; ++j) {
            const long Rj = s.bottoms[j] < 0 ? size : Rs[s.bottoms[j]];
            if (Rj != R) return at(i, "CONCAT bottoms differ in height / width");
            D += s.bottoms[j] < 0 ? depth : Ds[s.bottoms[j]];
          }
          break;
        case CCT_LAYER_RELU:
        case CCT_LAYER_SOFTMAXLOSS:
          break;
        default:
          return at(i, "unknown layer type " + std::to_string(s.type));
      }
      if ((s.type == CCT_LAYER_RELU || s.type == CCT_LAYER_DROPOUT) && b0 >= 0)
        for (int q = b0 + 1; q < i; ++q) {
          // in place on a tensor that an earlier layer already reads: that reader would see it change
          const cct_layer_spec &t = specs[q];
          const int nb = t.n_bottoms ? t.n_bottoms : 1;
          for (int j = 0; j < nb; ++j) {
            int tb = t.n_bottoms ? t.bottoms[j] : q - 1;
            while (tb >= 0 && (specs[tb].type == CCT_LAYER_RELU || specs[tb].type == CCT_LAYER_DROPOUT))
              tb = specs[tb].n_bottoms ? specs[tb].bottoms[0] : tb - 1;  // in-place layers write their bottom's tensor
            int mine = b0;
            while (mine >= 0 && (specs[mine].type == CCT_LAYER_RELU || specs[mine].type == CCT_LAYER_DROPOUT))
              mine = specs[mine].n_bottoms ? specs[mine].bottoms[0] : mine - 1;
            if (tb == mine && t.type != CCT_LAYER_RELU && t.type != CCT_LAYER_DROPOUT)
              return at(i, "runs in place on a tensor that layer " + std::to_string(q) + " already reads");
          }
        }
      Rs[i] = R;
      Ds[i] = D;
      if ((double)batch * (double)D * (double)R * (double)R >= 2147483648.0)
        return at(i, "output tensor has 2^31 elements or more");
    }
    return "";
  }

  Network(int batch, int depth, int size, const cct_layer_spec *specs, int n_specs, const cct_solver_param *sp)
      : batch_(batch) {
    try {
      build(depth, size, specs, n_specs, sp);
    } catch (...) {
      release();  // a constructor that throws runs no destructor: free what was built so far
      throw;
    }
  }

 private:
  void build(int depth, int size, const cct_layer_spec *specs, int n_specs, const cct_solver_param *sp) {
    const int batch = batch_;
    {
      const std::string why = validate(batch, depth, size, specs, n_specs, sp);
      if (!why.empty()) throw std::invalid_argument(why);
    }
    if (sp) {
      solver_.base_lr_ = sp->base_lr; solver_.momentum_ = sp->momentum; solver_.gamma_ = sp->gamma;
      solver_.power_ = sp->power; solver_.weight_decay_ = sp->weight_decay; solver_.stepsize_ = sp->stepsize;
      solver_.max_iter_ = sp->max_iter; solver_.random_seed_ = sp->random_seed;
      if (sp->lr_policy) solver_.lr_policy_ = sp->lr_policy;
      if (sp->regularization_type) solver_.regularization_type_ = sp->regularization_type;
    }
    labels_ = new CubeT(1, 1, 1, batch, &driver_);
    LayerT *const input_layer = new_layer(size, size, depth);
    blobs_[input_layer] = TensorInfo();
    for (int i = 0; i < n_specs; ++i) {
      nodes_.emplace_back();     // in place: what the node owns is freed by release() if a bridge below throws
      Node &nd = nodes_.back();  // (nothing else is appended to nodes_ during this iteration)
      nd.spec = specs[i];
      const cct_layer_spec &s = specs[i];
      // the tensor(s) this layer reads: the producers' layers as they are; `cur` becomes this node's
      // own view of the first one below (the same layer for the first reader and for in-place layers)
      std::vector<LayerT *> bottoms;
      if (s.n_bottoms == 0) bottoms.push_back(i == 0 ? input_layer : nodes_[i - 1].out);
      for (int j = 0; j < s.n_bottoms; ++j)
        bottoms.push_back(s.bottoms[j] < 0 ? input_layer : nodes_[s.bottoms[j]].out);
      const bool in_place = s.type == CCT_LAYER_RELU || s.type == CCT_LAYER_DROPOUT;
      bool params_upstream = false;
      for (LayerT *b : bottoms) params_upstream = params_upstream || blobs_[b].params_upstream;
      const bool first_weight_layer = !params_upstream;
      const int producer_node = blobs_[bottoms[0]].last_writer;  // -1: the network input
      for (LayerT *b : bottoms) nd.ins.push_back(in_place ? b : consume(b));
      LayerT *cur = nd.ins[0];
      nd.in = cur;
      const size_t R = cur->dR, D = cur->dD;
      switch (s.type) {
        case CCT_LAYER_CONV: {
          const int g = s.group > 1 ? s.group : 1;
          if (D % g || s.num_output % g) fail("group must divide input depth and num_output");
          const size_t m = (R + 2 * s.pad - s.kernel_size) / s.stride + 1;
          nd.out = new_layer(m, m, s.num_output);
          // A grouped layer whose geometry the direct kernels take is ONE bridge over the whole
          // tensors: the kernels run every group in the same launch.  Otherwise it is `g` bridges on
          // contiguous per-group layers, the slices gathered before and scattered after.
          const bool one_bridge = g > 1 && driver_.conv_direct_supported(batch_, (int)D, (int)R, s.kernel_size, s.stride,
                                                                         s.pad, s.num_output, g);
          const int n_bridges = one_bridge ? 1 : g;
          for (int gi = 0; gi < n_bridges; ++gi) {
            cnn::LayerParameter *lp = new_param(s);
            lp->convolution_param_.num_output_ = one_bridge ? s.num_output : s.num_output / g;
            lp->convolution_param_.group_ = one_bridge ? g : 1;
            lp->convolution_param_.kernel_size_ = s.kernel_size;
            lp->convolution_param_.stride_ = s.stride;
            lp->convolution_param_.pad_ = s.pad;
            lp->convolution_param_.bias_term_ = s.bias_term != 0;
            set_filler(lp->convolution_param_.weight_filler_, s.weight_filler);
            set_filler(lp->convolution_param_.bias_filler_, s.bias_filler);
            nd.params.push_back(lp);
            LayerT *gin = cur, *gout = nd.out;
            if (n_bridges > 1) {
              gin = new_layer(R, R, D / g);
              gout = new_layer(m, m, s.num_output / g);
              nd.group_in.push_back(gin);
              nd.group_out.push_back(gout);
            }
            auto *b = new ParallelizedBridge<float, ConvolutionBridge, HIPDriver>(gin, gout, lp, &solver_, &driver_);
            b->needs_to_calc_backward_grad = !first_weight_layer;
            nd.bridges.push_back(b);
          }
          break;
        }
        case CCT_LAYER_FC: {
          nd.out = new_layer(1, 1, s.num_output);
          cnn::LayerParameter *lp = new_param(s);
          lp->inner_product_param_.num_output_ = s.num_output;
          lp->inner_product_param_.bias_term_ = s.bias_term != 0;
          set_filler(lp->inner_product_param_.weight_filler_, s.weight_filler);
          set_filler(lp->inner_product_param_.bias_filler_, s.bias_filler);
          nd.params.push_back(lp);
          auto *b = new ParallelizedBridge<float, FullyConnectedBridge, HIPDriver>(cur, nd.out, lp, &solver_, &driver_);
          b->needs_to_calc_backward_grad = !first_weight_layer;
          nd.bridges.push_back(b);
          break;
        }
        case CCT_LAYER_RELU: {
          nd.out = cur;  // in place
          nd.params.push_back(new_param(s));
          auto *rb = new ReLUBridge<float, HIPDriver>(cur, cur, nd.params[0], &solver_, &driver_);
          // directly after a convolution the clamp rides on the convolution's output store (nothing
          // reads the tensor in between: an in-place layer on a tensor that already has readers is refused)
          if (producer_node >= 0 && nodes_[producer_node].spec.type == CCT_LAYER_CONV) {
            for (BridgeT *cb : nodes_[producer_node].bridges)
              static_cast<ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *>(cb)->sub_bridge()->set_fuse_relu(true);
            rb->forward_done_by_producer = true;
          } else if (producer_node >= 0 && nodes_[producer_node].spec.type == CCT_LAYER_FC) {
            // likewise after an inner-product layer: the clamp rides on the GEMM's output pass
            for (BridgeT *fb : nodes_[producer_node].bridges)
              static_cast<ParallelizedBridge<float, FullyConnectedBridge, HIPDriver> *>(fb)->sub_bridge()->set_fuse_relu(true);
            rb->forward_done_by_producer = true;
          }
          nd.bridges.push_back(rb);
          break;
        }
        case CCT_LAYER_DROPOUT: {
          nd.out = cur;  // in place
          cnn::LayerParameter *lp = new_param(s);
          lp->dropout_param_.dropout_ratio_ = s.dropout_ratio;
          nd.params.push_back(lp);
          nd.bridges.push_back(new DropoutBridge<float, HIPDriver>(cur, cur, lp, &solver_, &driver_));
          break;
        }
        case CCT_LAYER_MAXPOOL: {
          const size_t m = (R - s.kernel_size) / s.stride + 1;
          nd.out = new_layer(m, m, D);
          cnn::LayerParameter *lp = new_param(s);
          lp->pooling_param_.kernel_size_ = s.kernel_size;
          lp->pooling_param_.stride_ = s.stride;
          nd.params.push_back(lp);
          nd.bridges.push_back(new MaxPoolingBridge<float, HIPDriver>(cur, nd.out, lp, &solver_, &driver_));
          break;
        }
        case CCT_LAYER_LRN: {
          nd.out = new_layer(R, R, D);
          cnn::LayerParameter *lp = new_param(s);
          lp->lrn_param_.local_size_ = s.lrn_local_size;
          lp->lrn_param_.alpha_ = s.lrn_alpha;
          lp->lrn_param_.beta_ = s.lrn_beta;
          nd.params.push_back(lp);
          nd.bridges.push_back(new LRNBridge<float, HIPDriver>(cur, nd.out, lp, &solver_, &driver_));
          break;
        }
        case CCT_LAYER_SOFTMAXLOSS: {
          nd.out = new_layer(R, R, D);
          nd.params.push_back(new_param(s));
          softmax_ = new SoftmaxLossBridge<float, HIPDriver>(cur, nd.out, nd.params[0], &solver_, &driver_, labels_);
          softmax_node_runs_backward_ = params_upstream;
          softmax_->gradient_with_forward = params_upstream;  // chains start in the TRAIN phase
          nd.bridges.push_back(softmax_);
          break;
        }
        case CCT_LAYER_CONCAT: {
          size_t total_d = 0;
          for (LayerT *b : nd.ins) total_d += b->dD;
          nd.out = new_layer(R, R, total_d);
          break;
        }
        default:
          fail("unknown layer type");
      }
      const bool has_params = s.type == CCT_LAYER_CONV || s.type == CCT_LAYER_FC;
      nd.run_backward = has_params || params_upstream;
      TensorInfo &ob = blobs_[nd.out];  // created here for a new tensor, found for an in-place layer
      ob.params_upstream = ob.params_upstream || params_upstream || has_params;
      ob.last_writer = i;
      ob.writers.push_back(i);
    }
    // Fusions that depend on who reads a tensor, decided now that every reader is known.
    for (size_t i = 0; i < nodes_.size(); ++i) {
      Node &nd = nodes_[i];
      if (nd.spec.type == CCT_LAYER_FC) {
        // an inner-product layer of few outputs masks its input gradient in its one backward launch
        auto *fb = static_cast<ParallelizedBridge<float, FullyConnectedBridge, HIPDriver> *>(nd.bridges[0])->sub_bridge();
        if (!fb->small_kernels()) continue;
      } else if (nd.spec.type != CCT_LAYER_CONV && nd.spec.type != CCT_LAYER_MAXPOOL) {
        continue;
      }
      const cct_layer_spec &s = nd.spec;
      LayerT *bottom = s.n_bottoms ? (s.bottoms[0] < 0 ? layers_[0] : nodes_[s.bottoms[0]].out)
                                   : (i == 0 ? layers_[0] : nodes_[i - 1].out);
      const TensorInfo &bb = blobs_[bottom];
      // the last layer that wrote the tensor before this reader came
      int writer = -1;
      for (int w : bb.writers)
        if (w < (int)i) writer = w;
      // Directly after an in-place ReLU, and as the tensor's only reader, the layer performs that
      // ReLU's backward itself: a convolution masks the input gradient it produces (in the direct
      // kernel's store), a pooling layer stores its gradient already masked; the ReLU bridge then
      // skips its own backward pass over the tensor.
      if (writer >= 0 && nodes_[writer].spec.type == CCT_LAYER_RELU && bb.readers == 1 && bb.writers.back() == writer &&
          nd.bridges[0]->needs_to_calc_backward_grad && nd.run_backward) {
        if (nd.spec.type == CCT_LAYER_CONV)
          for (BridgeT *cb : nd.bridges)
            static_cast<ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *>(cb)->sub_bridge()->input_is_relu_output = true;
        else if (nd.spec.type == CCT_LAYER_FC)
          static_cast<ParallelizedBridge<float, FullyConnectedBridge, HIPDriver> *>(nd.bridges[0])->sub_bridge()->input_is_relu_output = true;
        else
          static_cast<MaxPoolingBridge<float, HIPDriver> *>(nd.bridges[0])->input_is_relu_output = true;
        static_cast<ReLUBridge<float, HIPDriver> *>(nodes_[writer].bridges[0])->backward_done_by_consumer = true;
      }
      if (nd.spec.type == CCT_LAYER_MAXPOOL) {
        // a pooling layer that folds a ReLU backward may take its mask from its own output, unless a
        // later layer rewrites that tensor in place (dropout does; a ReLU keeps the signs)
        bool rewritten = false;
        for (int w : blobs_[nd.out].writers)
          if (w > (int)i && nodes_[w].spec.type != CCT_LAYER_RELU) rewritten = true;
        static_cast<MaxPoolingBridge<float, HIPDriver> *>(nd.bridges[0])->output_keeps_signs = !rewritten;
      }
    }
  }

  void release() {
    for (void *t : fwd_timers_) if (t) cct_hip_timer_destroy(t);
    for (void *t : bwd_timers_) if (t) cct_hip_timer_destroy(t);
    if (update_timer_) cct_hip_timer_destroy(update_timer_);
    fwd_timers_.clear(); bwd_timers_.clear(); update_timer_ = nullptr;
    for (Node &nd : nodes_) {
      for (BridgeT *b : nd.bridges) delete b;
      for (cnn::LayerParameter *p : nd.params) delete p;
    }
    nodes_.clear();
    for (LayerT *l : layers_) delete l;
    layers_.clear();
    delete labels_;
    labels_ = nullptr;
  }

 public:
  ~Network() { release(); }
  Network(const Network &) = delete;
  Network &operator=(const Network &) = delete;

  float *input() { return layers_[0]->p_data_cube->get_p_data(); }
  float *labels() { return labels_->get_p_data(); }
  int num_layers() const { return (int)nodes_.size(); }
  Node &node(int i) { return nodes_[i]; }
  HIPDriver &driver() { return driver_; }

  void set_train(bool train) {
    for (Node &nd : nodes_)
      if (nd.spec.type == CCT_LAYER_DROPOUT)
        static_cast<DropoutBridge<float, HIPDriver> *>(nd.bridges[0])->train = train;
    // TRAIN phase: every forward pass is followed by a backward pass, so the loss layer writes its
    // gradient in the launch that computes the probabilities (if anything upstream wants one)
    if (softmax_) softmax_->gradient_with_forward = train && softmax_node_runs_backward_;
  }

  // Per-layer times of the passes that follow, from events on the library's stream (what the
  // reference prints per bridge from report_forward_history / report_backward_updateweight_history,
  // src/DeepNet.h:2190-2215, measured on the device instead of the host clock), plus the stage
  // timing of every convolution bridge.  Off by default: an event pair per layer costs launch slots.
  void set_profiling(bool on) {
    profile_ = on;
    if (on && fwd_timers_.empty()) {
      fwd_timers_.assign(nodes_.size(), nullptr);
      bwd_timers_.assign(nodes_.size(), nullptr);
      ran_fwd_.assign(nodes_.size(), false);
      ran_bwd_.assign(nodes_.size(), false);
    }
    for (Node &nd : nodes_)
      if (nd.spec.type == CCT_LAYER_CONV)
        for (BridgeT *b : nd.bridges)
          static_cast<ParallelizedBridge<float, ConvolutionBridge, HIPDriver> *>(b)->sub_bridge()->set_stage_profiling(on);
  }
  // milliseconds of layer i's last profiled forward / backward step (0 if it did not run); waits for the step
  float layer_ms(int i, bool backward) {
    std::vector<void *> &t = backward ? bwd_timers_ : fwd_timers_;
    std::vector<bool> &ran = backward ? ran_bwd_ : ran_fwd_;
    float ms = 0.f;
    if (i >= 0 && i < (int)t.size() && t[i] && ran[i]) cct_hip_timer_elapsed_ms(t[i], &ms);
    return ms;
  }
  // milliseconds of the deferred SGD updates at the end of the last profiled backward pass
  float update_ms() {
    float ms = 0.f;
    if (update_timer_ && ran_update_) cct_hip_timer_elapsed_ms(update_timer_, &ms);
    return ms;
  }

  // DeepNet::run_forward_pass: every bridge in order
  void forward() {
    for (size_t i = 0; i < nodes_.size(); ++i) {
      Node &nd = nodes_[i];
      tick(fwd_timers_, ran_fwd_, i, true);
      const size_t g = nd.group_in.size();
      for (size_t gi = 0; gi < g; ++gi)
        slice_copy(nd.group_in[gi]->p_data_cube, nd.in->p_data_cube, gi, /*gather=*/true);
      if (nd.spec.type == CCT_LAYER_CONCAT) concat_copy(nd, /*data=*/true);
      for (BridgeT *b : nd.bridges) b->forward();
      for (size_t gi = 0; gi < g; ++gi)
        slice_copy(nd.group_out[gi]->p_data_cube, nd.out->p_data_cube, gi, /*gather=*/false);
      tick(fwd_timers_, ran_fwd_, i, false);
    }
  }

  // DeepNet::run_backward_pass: every bridge in reverse order; ParallelizedBridge::backward applies
  // the SGD update of its layer
  void backward() {
    // the layers' SGD updates are collected and applied after the last backward: the many small
    // tensors then share one launch
    driver_.begin_deferred_sgd();
    for (auto &kv : blobs_) kv.second.summed = false;
    if (profile_) std::fill(ran_bwd_.begin(), ran_bwd_.end(), false);
    for (int i = (int)nodes_.size() - 1; i >= 0; --i) {
      Node &nd = nodes_[i];
      if (!nd.run_backward) continue;
      tick(bwd_timers_, ran_bwd_, i, true);
      sum_reader_gradients(nd.out);
      if (nd.spec.type == CCT_LAYER_CONCAT) {
        concat_copy(nd, /*data=*/false);
        tick(bwd_timers_, ran_bwd_, i, false);
        continue;
      }
      const size_t g = nd.group_in.size();
      for (size_t gi = 0; gi < g; ++gi)
        slice_copy(nd.group_out[gi]->p_gradient_cube, nd.out->p_gradient_cube, gi, /*gather=*/true);
      for (BridgeT *b : nd.bridges) b->backward();
      if (nd.bridges[0]->needs_to_calc_backward_grad)
        for (size_t gi = 0; gi < g; ++gi)
          slice_copy(nd.group_in[gi]->p_gradient_cube, nd.in->p_gradient_cube, gi, /*gather=*/false);
      tick(bwd_timers_, ran_bwd_, i, false);
    }
    if (profile_) {
      if (!update_timer_) cct_hip_timer_create(&update_timer_);
      cct_hip_timer_start(update_timer_);
    }
    driver_.flush_deferred_sgd();
    if (profile_) {
      cct_hip_timer_stop(update_timer_);
      ran_update_ = true;
    }
  }

  float loss() { return softmax_ ? softmax_->get_loss() : 0.f; }

  // ---- model files and snapshots (src/DeepNet.h:268-422) ----
  enum Blob { BLOB_MODEL, BLOB_HISTORY };
  const std::string &io_error() const { return io_error_; }

  // DeepNet::write_model_to_file / write_momentum_to_file
  bool write_blobs(const std::string &file, Blob what) {
    FILE *f = std::fopen(file.c_str(), "wb");
    if (!f) return io_fail("Error opening " + file);
    bool ok = true;
    std::vector<float> host;
    for_each_blob(what, [&](CubeT *c) {
      host.resize(c->n_elements);
      if (cct_hip_memcpy(host.data(), c->get_p_data(), host.size() * sizeof(float), 1)) fail(cct_hip_last_error());
      ok = ok && std::fwrite(host.data(), sizeof(float), host.size(), f) == host.size();
    });
    ok = (std::fclose(f) == 0) && ok;
    return ok ? true : io_fail("short write to " + file);
  }

  // DeepNet::read_model_from_file / read_momentum_from_file; the file must hold every blob
  bool read_blobs(const std::string &file, Blob what) {
    FILE *f = std::fopen(file.c_str(), "rb");
    if (!f) return io_fail("Error opening " + file);
    bool ok = true;
    std::vector<float> host;
    for_each_blob(what, [&](CubeT *c) {
      if (!ok) return;
      host.resize(c->n_elements);
      ok = std::fread(host.data(), sizeof(float), host.size(), f) == host.size();
      if (ok && cct_hip_memcpy(c->get_p_data(), host.data(), host.size() * sizeof(float), 0)) fail(cct_hip_last_error());
    });
    std::fclose(f);
    return ok ? true : io_fail(file + " holds fewer values than the network's blobs");
  }

  // DeepNet::get_parameter_size (src/DeepNet.h:425-441)
  size_t parameter_size() {
    size_t n = 0;
    for_each_blob(BLOB_MODEL, [&](CubeT *c) { n += c->n_elements; });
    return n;
  }

  void set_current_iter(int iter) {
    for (Node &nd : nodes_)
      for (BridgeT *b : nd.bridges) b->set_current_iter(iter);
  }
  // updates applied so far by the first layer that has a model (all updaters advance together)
  int current_iter() {
    for (Node &nd : nodes_)
      for (BridgeT *b : nd.bridges)
        if (b->get_current_iter() >= 0) return b->get_current_iter();
    return 0;
  }
  // scores per image entering the loss layer (0 without one): labels must lie in [0, this)
  int num_classes() const { return softmax_ ? (int)(softmax_->iR * softmax_->iC * softmax_->iD) : 0; }

  // DeepNet::write_full_snapshot (src/DeepNet.h:268-295)
  bool write_snapshot(const std::string &base_filename, int iter) {
    const std::string stem = base_filename + ".snapshot_iter" + std::to_string(iter);
    if (!write_blobs(stem + ".MODEL.bin", BLOB_MODEL) || !write_blobs(stem + ".HISTORY.bin", BLOB_HISTORY))
      return false;
    FILE *f = std::fopen((stem + ".ITER.bin").c_str(), "wb");
    if (!f) return io_fail("Error opening " + stem + ".ITER.bin");
    const bool ok = std::fwrite(&iter, sizeof(int), 1, f) == 1;
    return (std::fclose(f) == 0 && ok) ? true : io_fail("short write to " + stem + ".ITER.bin");
  }

  // DeepNet::read_full_snapshot (src/DeepNet.h:297-326); `stem` ends in ".snapshot_iter<N>"
  bool read_snapshot(const std::string &stem, int *iter_out) {
    if (!read_blobs(stem + ".MODEL.bin", BLOB_MODEL) || !read_blobs(stem + ".HISTORY.bin", BLOB_HISTORY))
      return false;
    FILE *f = std::fopen((stem + ".ITER.bin").c_str(), "rb");
    if (!f) return io_fail("Error opening " + stem + ".ITER.bin");
    int iter = 0;
    const bool ok = std::fread(&iter, sizeof(int), 1, f) == 1;
    std::fclose(f);
    if (!ok) return io_fail(stem + ".ITER.bin is empty");
    set_current_iter(iter);
    if (iter_out) *iter_out = iter;
    return true;
  }

 private:
  HIPDriver driver_;
  cnn::SolverParameter solver_;
  int batch_;
  CubeT *labels_ = nullptr;
  std::vector<LayerT *> layers_;
  std::vector<Node> nodes_;
  SoftmaxLossBridge<float, HIPDriver> *softmax_ = nullptr;
  bool softmax_node_runs_backward_ = false;

  // What the network knows about a tensor (a Layer that some node produced, or the input).
  struct TensorInfo {
    int readers = 0;                   // layers that read it (in-place layers do not count)
    std::vector<CubeT *> extra_grads;  // gradient cubes of the second, third, ... reader
    std::vector<int> writers;          // producer and in-place layers, in order
    int last_writer = -1;
    bool params_upstream = false;      // a layer with weights lies at or above its producer
    bool summed = false;               // reader gradients added up in the current backward pass
  };
  std::map<LayerT *, TensorInfo> blobs_;

  // A reader's view of tensor `L`: the layer itself for the first reader; for every further reader
  // the same data with a gradient cube of its own (the reference's Split: shared data, one
  // gradient per output, src/DeepNet.h:1924-2028).
  LayerT *consume(LayerT *L) {
    TensorInfo &b = blobs_[L];
    if (b.readers++ == 0) return L;
    LayerT *v = new LayerT(new CubeT(L->p_data_cube->get_p_data(), L->dR, L->dC, L->dD, batch_),
                           new CubeT(L->dR, L->dC, L->dD, batch_, &driver_));
    layers_.push_back(v);
    b.extra_grads.push_back(v->p_gradient_cube);
    return v;
  }
  // gradient of `L` = first reader's + second reader's + ... (ascending, fp32), once per backward pass
  void sum_reader_gradients(LayerT *L) {
    TensorInfo &b = blobs_[L];
    if (b.summed) return;
    b.summed = true;
    DeviceMemoryPointer total = L->p_gradient_cube->get_device_pointer(&driver_);
    for (CubeT *e : b.extra_grads) {
      DeviceMemoryPointer part = e->get_device_pointer(&driver_);
      driver_.math_saxpy(1.0f, &part, &total);
    }
  }
  // CONCAT: bottoms -> channel slices of the output (data, forward) or back (gradient, backward)
  void concat_copy(Node &nd, bool data) {
    size_t d_off = 0;
    for (LayerT *b : nd.ins) {
      CubeT *part = data ? b->p_data_cube : b->p_gradient_cube;
      CubeT *whole = data ? nd.out->p_data_cube : nd.out->p_gradient_cube;
      const int rc_ = cct_hip_copy_depth_slice(part->get_p_data(), whole->get_p_data(), (int)part->B, (int)whole->D,
                                               (int)d_off, (int)part->D, part->R * part->C, data ? 0 : 1);
      if (rc_) fail(cct_hip_last_error());
      d_off += part->D;
    }
  }

  bool profile_ = false, ran_update_ = false;
  std::vector<void *> fwd_timers_, bwd_timers_;
  std::vector<bool> ran_fwd_, ran_bwd_;
  void *update_timer_ = nullptr;
  void tick(std::vector<void *> &timers, std::vector<bool> &ran, size_t i, bool start) {
    if (!profile_) return;
    if (!timers[i]) cct_hip_timer_create(&timers[i]);
    if (start) {
      cct_hip_timer_start(timers[i]);
    } else {
      cct_hip_timer_stop(timers[i]);
      ran[i] = true;
    }
  }

  std::string io_error_;
  bool io_fail(const std::string &msg) {
    io_error_ = msg;
    return false;
  }
  // Bridges in order; per bridge model then bias (src/DeepNet.h:335-352).  The groups of a grouped
  // convolution are written as ONE layer -- all group models in order ([o][d/g][k][k]), then all
  // group biases ([o]) -- the blob layout such a layer has in Caffe; the reference ignores `group`.
  template <typename F>
  void for_each_blob(Blob what, F f) {
    for (Node &nd : nodes_) {
      for (BridgeT *b : nd.bridges)
        if (CubeT *c = what == BLOB_MODEL ? b->get_model_cube() : b->get_model_history_cube()) f(c);
      for (BridgeT *b : nd.bridges)
        if (CubeT *c = what == BLOB_MODEL ? b->get_bias_cube() : b->get_bias_history_cube()) f(c);
    }
  }
  static void set_filler(cnn::FillerParameter &dst, const cct_filler &src) {
    static const char *const names[] = {"constant", "xavier", "gaussian", "bernoulli"};
    if (src.type < 0 || src.type > 3) fail("unknown filler type");
    dst.type_ = names[src.type];
    dst.value_ = src.value; dst.mean_ = src.mean; dst.std_ = src.std;
  }
  // caught at the C boundary (cct_net_create and friends return an error code and message)
  [[noreturn]] static void fail(const char *msg) { throw std::runtime_error(std::string("Network: ") + msg); }
  LayerT *new_layer(size_t R, size_t C, size_t D) {
    LayerT *l = new LayerT(new CubeT(R, C, D, batch_, &driver_), new CubeT(R, C, D, batch_, &driver_));
    layers_.push_back(l);
    return l;
  }
  static cnn::LayerParameter *new_param(const cct_layer_spec &s) {
    cnn::LayerParameter *lp = new cnn::LayerParameter;
    lp->blobs_lr_[0] = s.lr_mult[0]; lp->blobs_lr_[1] = s.lr_mult[1];
    lp->weight_decay_[0] = s.decay_mult[0]; lp->weight_decay_[1] = s.decay_mult[1];
    return lp;
  }
  // part: [B][D/g][R][C] contiguous; whole: [B][D][R][C]; moves channel group gi
  void slice_copy(CubeT *part, CubeT *whole, size_t gi, bool gather) {
    const size_t rc = part->R * part->C;
    int rc_ = cct_hip_copy_depth_slice(part->get_p_data(), whole->get_p_data(), (int)part->B, (int)whole->D,
                                       (int)(gi * part->D), (int)part->D, rc, gather ? 1 : 0);
    if (rc_) fail(cct_hip_last_error());
  }
};

}  // namespace cct
