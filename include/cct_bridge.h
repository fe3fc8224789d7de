/*
 * cct_bridge.h -- C entry points over the C++ host layer (caffecontroll_amd/csrc/host/*.h) so that
 * the operator-level path can be driven and checked from any language with a C FFI.
 *
 * The reference's operators are C++ class templates, not an FFI; each function below stands for
 * one member of them on the HIP driver:
 *   ConvolutionBridge<float,...,DriverClass>::forward / backward
 *       src/bridges/ConvolutionBridge_impl.hxx:284-520, 541-796
 *   ParallelizedBridge<float, ConvolutionBridge>::forward / backward (one device partition,
 *   gradient update on the device)   src/bridges/ParallelizedBridge_impl.hxx:508-753, 761-1141
 *   SGDGradientUpdater::update        src/algorithms/GradientUpdater.h:154-193
 * All data pointers are device pointers.  Return value: 0 on success, non-zero otherwise
 * (cct_hip_last_error() has the text).  That includes failures inside the C++ layer (a HIP error
 * in the middle of an iteration, an inconsistent layer): a C++ caller of the bridges gets the
 * reference's abort-on-error, these entry points never end the caller's process.
 */
#ifndef CCT_BRIDGE_H
#define CCT_BRIDGE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* cnn::SolverParameter fields read on this path (src/parser/cnn.proto:56-160). */
typedef struct cct_solver_param {
  float base_lr, momentum, gamma, power, weight_decay;
  int stepsize, max_iter, random_seed;
  const char *lr_policy;           /* "fixed" "step" "exp" "inv" "poly" "sigmoid" */
  const char *regularization_type; /* "L2" or "L1" */
} cct_solver_param;

/* cnn::LayerParameter / ConvolutionParameter fields of a CONVOLUTION layer. */
typedef struct cct_conv_param {
  int num_output, kernel_size, stride, pad, bias_term;
  float lr_mult_weights, lr_mult_bias, decay_mult_weights, decay_mult_bias;
} cct_conv_param;

/* Stage order of cct_conv_bridge_stage_ms: the reference's detailed-profiling labels
 * "Lower Cube", "GEMM", "Remap", "Bias" (forward), "Bias", "Remap", "GEMM Data", "Inverse Lwr",
 * "GEMM Wghts" (backward) -- src/bridges/ConvolutionBridge_impl.hxx:325-366, 601-623. */
#define CCT_CONV_STAGE_COUNT 9

typedef struct cct_conv_bridge cct_conv_bridge;

/* Builds input/output layers over the caller's device buffers (in_data/in_grad [b][d][n][n],
 * out_data/out_grad [b][o][m][m]) and a ParallelizedBridge<ConvolutionBridge> on them.
 * Weights start at 0 and bias at 0 (constant fillers); write them through
 * cct_conv_bridge_model()/..._bias(). */
int cct_conv_bridge_create(cct_conv_bridge **out, int b, int d, int n, const cct_conv_param *conv,
                           const cct_solver_param *solver, float *in_data, float *in_grad, float *out_data,
                           float *out_grad);
/* The same with the reference's placement flags (src/bridges/ParallelizedBridge.h:183-198):
 * share_pointer_with_prev_bridge == 0 means in_data / in_grad are HOST arrays -- the bridge owns
 * device copies, uploads the input data in forward() and downloads the input gradient in
 * backward(), as the reference's bridge does when the previous bridge is not on the same device
 * (_impl.hxx:595-621, 686-705); share_pointer_with_next_bridge == 0 does the same for the output
 * layer.  With both flags 0 the bridge runs on plain host tensors, which is how the reference's
 * own bridge tests drive it (tests/test_parallelized_convolution.cpp:123-270). */
int cct_conv_bridge_create_shared(cct_conv_bridge **out, int b, int d, int n, const cct_conv_param *conv,
                                  const cct_solver_param *solver, float *in_data, float *in_grad, float *out_data,
                                  float *out_grad, int share_pointer_with_prev_bridge,
                                  int share_pointer_with_next_bridge);
int cct_conv_bridge_destroy(cct_conv_bridge *h);
/* fused: how much of the lowering pipeline is replaced.  0 = the reference's separate passes;
 * 1 = forward GEMM epilogue does remap + bias, bias gradient inside the lift launch; 2 = as 1 with
 * the data gradient from the direct-convolution kernel; 3 = forward and both gradients from direct
 * kernels, no lowered matrix.  2 and 3 fall back to 1 where cct_hip_conv_direct_supported() says
 * no.  A negative value keeps the bridge's default (3 where supported and the layer's
 * GEMMs are at least 2 GFLOP each, else 1).
 * profile: per-stage hipEvent timing; needs_backward_grad: compute the input gradient
 * (the first weight layer of a net does not, src/DeepNet.h:1108-1110). */
int cct_conv_bridge_set_options(cct_conv_bridge *h, int fused, int profile, int needs_backward_grad);
/* The level in effect (0..3, see above). */
int cct_conv_bridge_path(cct_conv_bridge *h);
/* Host-resident layers (cct_conv_bridge_create_shared with a share flag 0): overlapped != 0 (the default)
 * moves the batch in four pieces through two copy streams, piece i+1 uploading and piece i-1 downloading
 * while piece i computes, when the layer runs on its all-direct path; 0 is the reference's sequence of
 * one blocking copy in, the pass, one blocking copy out (src/bridges/ParallelizedBridge_impl.hxx:595-621,
 * 686-705).  Same results bit for bit.  cct_conv_bridge_staging: 1 if forward/backward will run in pieces. */
int cct_conv_bridge_set_staging(cct_conv_bridge *h, int overlapped);
/* ParallelizedBridge::set_share_pointer_with_next_bridge(true) (src/bridges/ParallelizedBridge.h:190-194), which
 * the builder of the NEXT bridge calls once it knows that bridge lives on the same device (src/DeepNet.h:1116-1120):
 * a bridge created with share_pointer_with_next_bridge == 0 stops copying its output to the host; its output layer
 * becomes the given DEVICE tensors (out_data / out_grad [b][o][m][m]), shared with the next bridge.  The flag
 * cannot be lowered again. */
int cct_conv_bridge_share_with_next(cct_conv_bridge *h, float *out_data_device, float *out_grad_device);
int cct_conv_bridge_staging(cct_conv_bridge *h);
float *cct_conv_bridge_model(cct_conv_bridge *h);      /* [o][d][k][k] */
float *cct_conv_bridge_bias(cct_conv_bridge *h);       /* [o] or NULL */
float *cct_conv_bridge_model_grad(cct_conv_bridge *h);
float *cct_conv_bridge_bias_grad(cct_conv_bridge *h);
float *cct_conv_bridge_lowered(cct_conv_bridge *h);    /* [b*m*m][k*k*d], valid after forward (levels 0-2) */
float *cct_conv_bridge_history(cct_conv_bridge *h);    /* momentum buffer of the weights */
int cct_conv_bridge_forward(cct_conv_bridge *h);
/* with_update != 0: ParallelizedBridge::backward (gradients, then SGD on weights and bias);
 * with_update == 0: ConvolutionBridge::backward only. */
int cct_conv_bridge_backward(cct_conv_bridge *h, int with_update);
int cct_conv_bridge_stage_ms(cct_conv_bridge *h, float ms[CCT_CONV_STAGE_COUNT]);
/* The kernel instance that ran as the stage's product kernel (cct_hip_last_kernel() taken when the
 * stage ended; needs profile != 0), "" for a stage that has not run.  Valid until the next
 * forward/backward of the bridge. */
const char *cct_conv_bridge_stage_kernel(cct_conv_bridge *h, int stage);

/* ---- a chain of layers (LeNet / CaffeNet style) --------------------------------------------
 * Stands for DeepNet::construct_network + run_forward_pass / run_backward_pass
 * (src/DeepNet.h:968-2030, 171-266): layers in the order the prototxt lists them (a topological
 * order), each reading the previous one or the layers its `bottoms` name, every layer wrapped in
 * a one-partition ParallelizedBridge on the device. */
enum cct_layer_type {
  CCT_LAYER_CONV = 1, CCT_LAYER_FC = 2, CCT_LAYER_RELU = 3, CCT_LAYER_MAXPOOL = 4, CCT_LAYER_LRN = 5,
  CCT_LAYER_DROPOUT = 6, CCT_LAYER_SOFTMAXLOSS = 7,
  CCT_LAYER_CONCAT = 8 /* depth-wise concatenation of 2..CCT_MAX_BOTTOMS bottoms (src/DeepNet.h:1700-1757) */
};
#define CCT_MAX_BOTTOMS 4

/* cnn::FillerParameter (src/parser/cnn.proto:21-32).  A zeroed struct is the proto default for
 * type and value ("constant", 0); set std explicitly for a gaussian filler (proto default 1). */
enum cct_filler_type { CCT_FILLER_CONSTANT = 0, CCT_FILLER_XAVIER = 1, CCT_FILLER_GAUSSIAN = 2, CCT_FILLER_BERNOULLI = 3 };
typedef struct cct_filler {
  int type;          /* enum cct_filler_type */
  float value;       /* constant: the value; bernoulli: the probability */
  float mean, std;   /* gaussian */
} cct_filler;

/* The fields of cnn::LayerParameter this path reads; unused ones are ignored per type. */
typedef struct cct_layer_spec {
  int type;                 /* enum cct_layer_type */
  int num_output;           /* conv, fc */
  int kernel_size, stride, pad; /* conv, pooling */
  int group;                /* conv: independent channel groups (<= 1: none) */
  int bias_term;            /* conv, fc */
  int lrn_local_size;
  float lrn_alpha, lrn_beta;
  float dropout_ratio;
  float lr_mult[2];         /* weights, bias */
  float decay_mult[2];
  cct_filler weight_filler, bias_filler; /* conv, fc; random fillers draw from solver.random_seed */
  /* Where the layer reads from.  n_bottoms == 0: the output of the previous layer in the array (the
   * network input for layer 0) -- a plain chain.  Otherwise bottoms[j] is the index of the layer
   * whose output is read, or -1 for the network input; every layer but CONCAT has one bottom.  A
   * layer output read by several layers is the reference's Split (src/DeepNet.h:1924-2028): the
   * readers share the data, each writes a gradient of its own, and the gradients are added up, in
   * reader order, before the producer's backward step. */
  int n_bottoms;
  int bottoms[CCT_MAX_BOTTOMS];
} cct_layer_spec;

typedef struct cct_net cct_net;

/* Checks a description the way cct_net_create does, on the host only (no device is touched):
 * positive sizes, stride >= 1, 1 <= kernel_size <= (padded) input, num_output >= 1, group divides
 * both depths, odd LRN window, dropout_ratio in [0, 1), known filler / layer / lr_policy names,
 * tensors below 2^31 elements.  The reference asserts or divides by zero on such input
 * (src/DeepNet.h:112-115, 1374-1376); here the call returns CCT_HIP_EINVAL and
 * cct_hip_last_error() names the layer. */
int cct_net_validate(int batch, int depth, int size, const cct_layer_spec *layers, int n_layers,
                     const cct_solver_param *solver);
int cct_net_create(cct_net **out, int batch, int depth, int size, const cct_layer_spec *layers, int n_layers,
                   const cct_solver_param *solver);
int cct_net_destroy(cct_net *net);
float *cct_net_input(cct_net *net);   /* device [batch][depth][size][size] */
float *cct_net_labels(cct_net *net);  /* device, one float per image */
int cct_net_num_layers(cct_net *net);
/* Device pointer + element count of a tensor of layer `layer`, channel group `group`:
 * which = 0 model, 1 bias, 2 model gradient, 3 bias gradient, 4 output data of the layer,
 * 5 gradient w.r.t. the layer's input, 6 dropout mask (uint32) / max-pool argmax (int32),
 * 7 momentum buffer of the model, 8 momentum buffer of the bias.  For a grouped convolution 0-3, 7
 * and 8 are the group's own [o/g][d/g][k][k] / [o/g] slices.
 * Returns NULL (and *n = 0) when the layer has no such tensor. */
void *cct_net_tensor(cct_net *net, int layer, int group, int which, size_t *n);
int cct_net_set_train(cct_net *net, int train);
/* Keep the dropout masks as they are instead of drawing new ones (for parity tests). */
int cct_net_freeze_dropout_masks(cct_net *net, int freeze);
/* Path level of every convolution layer (0 staged passes .. 3 all direct, as cct_conv_layer_set_options;
 * a layer falls back where the direct kernels do not cover its geometry, and a grouped layer, which
 * works on channel slices, stays on the direct kernels).  -1 puts every layer back on its default.
 * Without a counterpart in the reference: it is how tests run one network on every path. */
int cct_net_set_conv_path(cct_net *net, int level);
int cct_net_forward(cct_net *net);
int cct_net_backward(cct_net *net);   /* gradients + SGD update of every layer */
int cct_net_loss(cct_net *net, float *loss_sum); /* batch-summed loss of the last forward (syncs) */
/* Per-layer device times of the forward / backward passes that follow (events on the library's stream
 * around every layer; the reference prints the same breakdown from its per-bridge reports,
 * src/DeepNet.h:2190-2215, src/bridges/ConvolutionBridge_impl.hxx:325-366) and stage timing of every
 * convolution bridge.  Off by default.  cct_net_layer_ms waits for the layer's step and returns the
 * milliseconds of its last profiled forward and backward step (0 for a step that did not run; either
 * pointer may be NULL); cct_net_update_ms the deferred SGD updates at the end of the backward pass. */
int cct_net_set_profiling(cct_net *net, int on);
int cct_net_layer_ms(cct_net *net, int layer, float *forward_ms, float *backward_ms);
int cct_net_update_ms(cct_net *net, float *ms);
/* Convolution layers: number of bridges the layer runs as (1; `group` of them for a grouped layer whose
 * geometry the direct kernels do not take; 0 for other layer types), and per bridge what
 * cct_conv_bridge_stage_ms / _stage_kernel return for a single bridge. */
int cct_net_conv_bridges(cct_net *net, int layer);
int cct_net_conv_stage_ms(cct_net *net, int layer, int bridge, float ms[CCT_CONV_STAGE_COUNT]);
const char *cct_net_conv_stage_kernel(cct_net *net, int layer, int bridge, int stage);

/* Model files and snapshots in the reference's format: raw fp32, per bridge its model then its
 * bias (DeepNet::write_model_to_file / read_model_from_file, src/DeepNet.h:328-374; the
 * `-output-model-file` / `-input-model-file` options of `caffe-ct`).  The groups of a grouped
 * convolution are stored as one layer: [o][d/g][k][k] then [o]. */
int cct_net_write_model(cct_net *net, const char *file);
int cct_net_read_model(cct_net *net, const char *file);
/* DeepNet::write_full_snapshot (src/DeepNet.h:268-295): writes
 * <base>.snapshot_iter<iter>.MODEL.bin, .HISTORY.bin (momentum buffers) and .ITER.bin (one int). */
int cct_net_write_snapshot(cct_net *net, const char *base_filename, int iter);
/* DeepNet::read_full_snapshot (src/DeepNet.h:297-326): `stem` is the common prefix of the three
 * files (ends in ".snapshot_iter<N>"); restores weights, momentum and the updaters' iteration
 * counter, which is also returned through *iter. */
int cct_net_read_snapshot(cct_net *net, const char *stem, int *iter);
/* Iteration counter of every gradient updater (learning-rate schedule position). */
int cct_net_set_iter(cct_net *net, int iter);
/* Updates applied so far (GradientUpdater::current_iter, src/algorithms/GradientUpdater.h:24,156). */
int cct_net_get_iter(cct_net *net);
/* Scores per image entering the SoftmaxWithLoss layer (0 without one): every label must lie in
 * [0, this) -- the loss indexes the scores with it (src/kernels/softmax.hxx:49-52). */
int cct_net_num_classes(cct_net *net);
/* Util::get_learning_rate (src/util.h:76-93) for the solver's policy at iteration `iter`: the value
 * SGDGradientUpdater::get_stepsize multiplies with the layer's lr_mult
 * (src/algorithms/GradientUpdater.h:42-45).  Host arithmetic only.  NaN for a policy the reference
 * rejects ("multistep", unknown names). */
float cct_solver_learning_rate(const cct_solver_param *solver, int iter);
/* DeepNet::get_parameter_size (src/DeepNet.h:425-441): weights + biases of all layers. */
size_t cct_net_parameter_size(cct_net *net);

#ifdef __cplusplus
}
#endif
#endif
