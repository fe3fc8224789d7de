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
 * (cct_hip_last_error() has the text).  Errors inside the C++ layer abort, as the reference's
 * asserts do.
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
int cct_conv_bridge_destroy(cct_conv_bridge *h);
/* fused: single-GEMM forward epilogue + bias gradient inside the lift launch (default 1);
 * profile: per-stage hipEvent timing; needs_backward_grad: compute the input gradient
 * (the first weight layer of a net does not, src/DeepNet.h:1108-1110). */
int cct_conv_bridge_set_options(cct_conv_bridge *h, int fused, int profile, int needs_backward_grad);
float *cct_conv_bridge_model(cct_conv_bridge *h);      /* [o][d][k][k] */
float *cct_conv_bridge_bias(cct_conv_bridge *h);       /* [o] or NULL */
float *cct_conv_bridge_model_grad(cct_conv_bridge *h);
float *cct_conv_bridge_bias_grad(cct_conv_bridge *h);
float *cct_conv_bridge_lowered(cct_conv_bridge *h);    /* [b*m*m][k*k*d], valid after forward */
float *cct_conv_bridge_history(cct_conv_bridge *h);    /* momentum buffer of the weights */
int cct_conv_bridge_forward(cct_conv_bridge *h);
/* with_update != 0: ParallelizedBridge::backward (gradients, then SGD on weights and bias);
 * with_update == 0: ConvolutionBridge::backward only. */
int cct_conv_bridge_backward(cct_conv_bridge *h, int with_update);
int cct_conv_bridge_stage_ms(cct_conv_bridge *h, float ms[CCT_CONV_STAGE_COUNT]);

#ifdef __cplusplus
}
#endif
#endif
