/*
 * CPU oracle for the lowering-based convolution training path of CaffeConTroll.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic that
 * CaffeConTroll's CPUDriver performs for the path; it exists to check the HIP
 * library and to time a CPU baseline.  Nothing in the product library links,
 * loads or calls it.
 *
 * Every function cites the reference file:line whose algorithm it restates
 * (paths relative to the CaffeConTroll source tree).
 *
 * Pinning status (what independent evidence fixes each function; the tests that
 * carry the evidence live in tests/test_oracle_*.py):
 *   lower_cube            worked matrices of docs/lowering/type_1/type_1_lowering_pad_stride.tex,
 *                         brute-force definition, conv fixtures (through conv_forward)
 *   remap                 closed form (slice permutation), conv fixtures
 *   sgemm / sgemm_new     numpy float64 matmul for every (order, TA, TB), conv fixtures
 *   sgemv                 numpy
 *   bias_forward/backward closed form, conv fixtures (conv_bias.txt)
 *   inverse_lower_cube    adjoint identity <lower(x),y> = <x,lift(y)>, brute force,
 *                         conv_backward fixtures
 *   conv_forward/backward reference fixtures tests/input/conv_* -> tests/output/conv_*
 *                         (small: exact integer arithmetic; large: 1e-3 as the reference test)
 *   sgd_update            fixtures conv_weights.txt / conv_bias.txt, 3-line recurrence
 *   relu, maxpool, dropout, softmax   reference fixtures (relu_*, pooling_*, dropout_*, softmax_*)
 *   lrn_forward/backward  reference fixtures lrn_* at 1e-3 (the fixtures were produced by a
 *                         build using an approximate pow; this oracle uses exact powf)
 *   process_image         numpy slicing formulation (window slice, [..., ::-1] for the mirror) on
 *                         random shapes; the reference holds no fixture for it
 *   fillers (mt19937 streams)         not restated; configs inject their own tensors
 */
#ifndef CCT_ORACLE_H
#define CCT_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same field order as struct PMapHelper, src/sched/DeviceHeader.h:25-35. */
typedef struct {
  size_t dR, dC, dD, dB;
  size_t sR, sC, sD, sB;
  size_t dBR, dBC;
  size_t sBR, sBC;
  size_t kR, kC, kD, kB;
  size_t stride;
  size_t padding;
} cct_oracle_pmap;

/* Same field order as struct _inverse_lower_cube_arg_helper, src/kernels/lowering.h:22-32. */
typedef struct {
  size_t data_output_width;
  size_t data_output_height;
  size_t kernel_size;
  size_t stride;
  size_t padding;
  size_t iR, iC, iD, iB;
} cct_oracle_lift_args;

enum { CCT_ROW_MAJOR = 101, CCT_COL_MAJOR = 102, CCT_NO_TRANS = 111, CCT_TRANS = 112 };

/* --- lowering / lifting / remap ------------------------------------------------ */
void cct_oracle_lower_cube(float *dst, const float *src, const cct_oracle_pmap *a);
void cct_oracle_inverse_lower_cube(float *dst, const float *src, const cct_oracle_lift_args *a);
void cct_oracle_remap(float *dst, const float *src, const cct_oracle_pmap *a);

/* --- BLAS-shaped pieces ---------------------------------------------------------- */
void cct_oracle_sgemm(int order, int TA, int TB, int M, int N, int K, float alpha,
                      const float *A, int lda, const float *B, int ldb, float beta,
                      float *C, int ldc);
/* Same contract, products and sums carried in double (arbitration reference). */
void cct_oracle_sgemm_f64acc(int order, int TA, int TB, int M, int N, int K, float alpha,
                             const float *A, int lda, const float *B, int ldb, float beta,
                             float *C, int ldc);
void cct_oracle_sgemm_new(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                          const float *B, float beta, float *C);
void cct_oracle_sgemv(int TA, int M, int N, float alpha, const float *A, const float *x,
                      float beta, float *y);
void cct_oracle_saxpy(size_t n, float alpha, const float *x, float *y);
void cct_oracle_saxpby(size_t n, float alpha, const float *x, float beta, float *y);
/* Route cct_oracle_sgemm through an OpenBLAS found at run time (CPU baseline only).
 * Returns 1 when a cblas_sgemm was bound, 0 when the naive loops stay in use. */
int cct_oracle_bind_openblas(const char *path, int nthreads);
int cct_oracle_blas_is_bound(void);

/* --- conv bias ------------------------------------------------------------------- */
void cct_oracle_bias_forward(float *out, const float *bias, size_t fmap, size_t depth, size_t batch);
void cct_oracle_bias_backward(float *bias_grad, const float *out_grad, size_t fmap, size_t depth,
                              size_t batch);

/* --- whole convolution (CPU branch of ConvolutionBridge) -------------------------- */
typedef struct {
  size_t b, d, n, k, s, p, o; /* m is derived */
} cct_oracle_conv_shape;
size_t cct_oracle_conv_m(const cct_oracle_conv_shape *c);
/* lowered: caller buffer of b*m*m*k*k*d floats, filled here and reused by backward */
void cct_oracle_conv_forward(const cct_oracle_conv_shape *c, const float *in, const float *model,
                             const float *bias /* may be NULL */, float *lowered, float *out);
/* out_grad is permuted in place to [o][b][m*m] exactly as the reference does.
 * lowered_grad: scratch of the same size as lowered (only touched if need_in_grad). */
void cct_oracle_conv_backward(const cct_oracle_conv_shape *c, const float *model,
                              float *out_grad, const float *lowered, float *lowered_grad,
                              float *in_grad /* may be NULL */, float *model_grad,
                              float *bias_grad /* may be NULL */, int need_in_grad);

/* --- SGD ------------------------------------------------------------------------- */
void cct_oracle_sgd_update(size_t n, float *model, float *grad, float *history, float stepsize,
                           float momentum, float lambda, int l1);
float cct_oracle_learning_rate(const char *policy, float base_lr, float gamma, float iter,
                               float stepsize, float power, float max_iter);

/* --- elementwise / pooling / loss -------------------------------------------------- */
void cct_oracle_relu_forward(float *out, const float *in, size_t n);
void cct_oracle_relu_backward(float *in_grad, const float *out_grad, const float *in_data, size_t n);
void cct_oracle_maxpool_forward(float *out, int *max_index, const float *in, int k, int s, int iR,
                                int iC, int oR, int oC, int D, int B);
void cct_oracle_maxpool_backward(float *in_grad, const float *out_grad, const int *max_index,
                                 int iR, int iC, int oR, int oC, int D, int B);
void cct_oracle_lrn_forward(float *out, float *denoms, const float *in, int iR, int iC, int iD,
                            int iB, int local_size, float alpha, float beta);
void cct_oracle_lrn_backward(float *in_grad, const float *out_grad, const float *in_data,
                             const float *denoms, int R, int C, int D, int B, int local_size,
                             float alpha, float beta);
void cct_oracle_dropout_forward(float *out, const float *in, const unsigned int *mask, float ratio,
                                size_t n);
void cct_oracle_dropout_forward_threshold(float *out, const float *in, const unsigned int *mask,
                                          float ratio, size_t n);
float cct_oracle_softmax_loss_forward(float *prob, const float *in, const float *labels, size_t iR,
                                      size_t iC, size_t iD, size_t iB);
void cct_oracle_softmax_loss_backward(float *in_grad, const float *prob, const float *labels,
                                      size_t iR, size_t iC, size_t iD, size_t iB);

/* --- fully connected (FullyConnectedBridge, sgemm_new path) ----------------------- */
void cct_oracle_fc_forward(float *out, const float *in, const float *model, const float *bias,
                           int B, int I, int O);
void cct_oracle_fc_backward(float *in_grad, float *model_grad, float *bias_grad, const float *in,
                            const float *model, const float *out_grad, int B, int I, int O,
                            int need_in_grad);

/* --- input transform (Corpus::process_image, src/parser/corpus.h:262-333) ---------- */
void cct_oracle_process_image(float *out, const unsigned char *data, const float *mean, int channels,
                              int height, int width, int crop_size, int h_off, int w_off, int mirror,
                              float scale);

#ifdef __cplusplus
}
#endif
#endif
