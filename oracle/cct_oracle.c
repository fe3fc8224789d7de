/*
 * CPU oracle (test infrastructure only) -- see cct_oracle.h for scope and pinning status.
 * Plain C99, built with -O2 and without -ffast-math so that the floating-point
 * evaluation order written here is the one executed.
 */
#include "cct_oracle.h"

#include <dlfcn.h>
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------
 * Type-1 lowering.  Restates CPUDriver::lower_cube (src/sched/DeviceDriver_CPU.cpp:124-301),
 * i.e. equation 4 of docs/lowering/type_1/type_1_lowering_pad_stride.tex:99-108:
 *   Dhat[(bi*m*m + r*m + c)*k*k*d + Dd*k*k + Dr*k + Dc]
 *       = D[bi*n*n*d + Dd*n*n + (r*s-p+Dr)*n + (c*s-p+Dc)]   (0 outside the image)
 * The reference blocks the Dd loop by 8; that only changes the visiting order of a pure copy.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_lower_cube(float *dst, const float *src, const cct_oracle_pmap *a) {
  const long n = (long)a->sR, d = (long)a->sD, k = (long)a->kR, s = (long)a->stride;
  const long p = (long)a->padding, b = (long)a->sB;
  const long m = (n + 2 * p - k) / s + 1;
  for (long bi = 0; bi < b; ++bi)
    for (long r = 0; r < m; ++r)
      for (long c = 0; c < m; ++c) {
        float *row = dst + ((bi * m + r) * m + c) * k * k * d;
        for (long dd = 0; dd < d; ++dd) {
          const float *plane = src + (bi * d + dd) * n * n;
          for (long kr = 0; kr < k; ++kr) {
            const long y = r * s - p + kr;
            float *seg = row + (dd * k + kr) * k;
            if (y < 0 || y >= n) {
              for (long kc = 0; kc < k; ++kc) seg[kc] = 0.0f;
              continue;
            }
            for (long kc = 0; kc < k; ++kc) {
              const long x = c * s - p + kc;
              seg[kc] = (x >= 0 && x < n) ? plane[y * n + x] : 0.0f;
            }
          }
        }
      }
}

/* ------------------------------------------------------------------------------------
 * Lifting (col2im scatter-add).  Restates CPUDriver::inverse_lower_cube
 * (src/sched/DeviceDriver_CPU.cpp:306-346) with the same loop nest id, ib, kr, cr, kc, cc so
 * that every destination pixel receives its addends in the same order (kr ascending, then kc
 * ascending).  dst is NOT cleared here: the caller zero-fills it first, as
 * Connector::inverse_lower_cube does (src/Connector_impl_Lowering_type1.hxx:156).
 * src layout: [iD*k*k][iB][oh*ow].
 * ---------------------------------------------------------------------------------- */
void cct_oracle_inverse_lower_cube(float *dst, const float *src, const cct_oracle_lift_args *a) {
  const size_t ow = a->data_output_width, oh = a->data_output_height;
  const size_t k = a->kernel_size, s = a->stride, p = a->padding;
  const size_t iR = a->iR, iC = a->iC, iD = a->iD, iB = a->iB;
  const size_t plane = iB * oh * ow;
  for (size_t id = 0; id < iD; ++id)
    for (size_t ib = 0; ib < iB; ++ib)
      for (size_t kr = 0; kr < k; ++kr)
        for (size_t cr = 0; cr < ow; ++cr) {
          const size_t y = cr * s + kr - p; /* wraps below zero -> fails the < iR test */
          if (!(y < iR)) continue;
          for (size_t kc = 0; kc < k; ++kc) {
            const float *srow = src + ((id * k + kr) * k + kc) * plane + ib * oh * ow + oh * cr;
            float *drow = dst + (ib * iD + id) * iR * iC + y * iC;
            for (size_t cc = 0; cc < oh; ++cc) {
              const size_t x = cc * s + kc - p;
              if (x < iC) drow[x] += srow[cc];
            }
          }
        }
}

/* ------------------------------------------------------------------------------------
 * Slice permutation.  Restates pmap2d_read_coalesce<_fpmap_id,_fmap_remap>
 * (src/sched/DeviceDriver_CPU.cpp:38-109 with src/kernels/lowering.hxx:241-258): source slice
 * j = id + ib*sD (sR x sC floats) lands at slice (j / sB) + (j % sB) * sD of the destination.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_remap(float *dst, const float *src, const cct_oracle_pmap *a) {
  const size_t R = a->sR, C = a->sC, D = a->sD, B = a->sB, rc = R * C;
  for (size_t j = 0; j < D * B; ++j) {
    const size_t reald = j / B, realb = j % B;
    memcpy(dst + (reald + realb * D) * rc, src + j * rc, rc * sizeof(float));
  }
}

/* ------------------------------------------------------------------------------------
 * GEMM with the cblas_sgemm contract, as called by CPUDriver::sgemm / sgemm_new
 * (src/sched/DeviceDriver_CPU.cpp:547-566).  The arithmetic itself lives in OpenBLAS
 * (third-party; the reference recommends OpenBLAS 0.2.14, README.md:188-192); what is restated
 * here is the published BLAS definition C = alpha*op(A)*op(B) + beta*C with fp32 products
 * summed in ascending k.
 * ---------------------------------------------------------------------------------- */
typedef void (*cblas_sgemm_fn)(int, int, int, int, int, int, float, const float *, int,
                               const float *, int, float, float *, int);
typedef void (*blas_threads_fn)(int);
static cblas_sgemm_fn g_blas_sgemm = NULL;

int cct_oracle_bind_openblas(const char *path, int nthreads) {
  if (path == NULL) {
    g_blas_sgemm = NULL;
    return 0;
  }
  void *h = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
  if (!h) return 0;
  cblas_sgemm_fn f = (cblas_sgemm_fn)dlsym(h, "scipy_cblas_sgemm");
  if (!f) f = (cblas_sgemm_fn)dlsym(h, "cblas_sgemm");
  if (!f) return 0;
  blas_threads_fn t = (blas_threads_fn)dlsym(h, "scipy_openblas_set_num_threads");
  if (!t) t = (blas_threads_fn)dlsym(h, "openblas_set_num_threads");
  if (t && nthreads > 0) t(nthreads);
  g_blas_sgemm = f;
  return 1;
}
int cct_oracle_blas_is_bound(void) { return g_blas_sgemm != NULL; }

static void gemm_generic(int order, int TA, int TB, int M, int N, int K, float alpha,
                         const float *A, int lda, const float *B, int ldb, float beta, float *C,
                         int ldc, int f64) {
  if (order == CCT_COL_MAJOR) { /* C^T = op(B)^T op(A)^T in row-major terms */
    gemm_generic(CCT_ROW_MAJOR, TB, TA, N, M, K, alpha, B, ldb, A, lda, beta, C, ldc, f64);
    return;
  }
  const long sai = (TA == CCT_NO_TRANS) ? lda : 1, sak = (TA == CCT_NO_TRANS) ? 1 : lda;
  const long sbk = (TB == CCT_NO_TRANS) ? ldb : 1, sbj = (TB == CCT_NO_TRANS) ? 1 : ldb;
  for (long i = 0; i < M; ++i)
    for (long j = 0; j < N; ++j) {
      float out;
      if (f64) {
        double acc = 0.0;
        for (long kk = 0; kk < K; ++kk)
          acc += (double)A[i * sai + kk * sak] * (double)B[kk * sbk + j * sbj];
        const double prev = (beta == 0.0f) ? 0.0 : (double)beta * (double)C[i * (long)ldc + j];
        out = (float)((double)alpha * acc + prev);
      } else {
        float acc = 0.0f;
        for (long kk = 0; kk < K; ++kk) acc += A[i * sai + kk * sak] * B[kk * sbk + j * sbj];
        out = (beta == 0.0f) ? alpha * acc : alpha * acc + beta * C[i * (long)ldc + j];
      }
      C[i * (long)ldc + j] = out;
    }
}

void cct_oracle_sgemm(int order, int TA, int TB, int M, int N, int K, float alpha, const float *A,
                      int lda, const float *B, int ldb, float beta, float *C, int ldc) {
  if (g_blas_sgemm) {
    g_blas_sgemm(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    return;
  }
  gemm_generic(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, 0);
}

void cct_oracle_sgemm_f64acc(int order, int TA, int TB, int M, int N, int K, float alpha,
                             const float *A, int lda, const float *B, int ldb, float beta,
                             float *C, int ldc) {
  gemm_generic(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, 1);
}

/* CPUDriver::sgemm_new, src/sched/DeviceDriver_CPU.cpp:557-566: row-major, implied strides. */
void cct_oracle_sgemm_new(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                          const float *B, float beta, float *C) {
  const int lda = (TA == CCT_NO_TRANS) ? K : M;
  const int ldb = (TB == CCT_NO_TRANS) ? N : K;
  cct_oracle_sgemm(CCT_ROW_MAJOR, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, C, N);
}

/* CPUDriver::sgemv, src/sched/DeviceDriver_CPU.cpp:568-574: row-major M x N matrix, lda = N. */
void cct_oracle_sgemv(int TA, int M, int N, float alpha, const float *A, const float *x,
                      float beta, float *y) {
  const int ylen = (TA == CCT_NO_TRANS) ? M : N, xlen = (TA == CCT_NO_TRANS) ? N : M;
  for (int i = 0; i < ylen; ++i) {
    float acc = 0.0f;
    for (int j = 0; j < xlen; ++j)
      acc += ((TA == CCT_NO_TRANS) ? A[(long)i * N + j] : A[(long)j * N + i]) * x[j];
    y[i] = (beta == 0.0f) ? alpha * acc : alpha * acc + beta * y[i];
  }
}

/* CPUDriver::math_saxpy / math_saxpby, src/sched/DeviceDriver_CPU.cpp:508-533 (vanilla loop). */
void cct_oracle_saxpby(size_t n, float alpha, const float *x, float beta, float *y) {
  for (size_t i = 0; i < n; ++i) y[i] = alpha * x[i] + beta * y[i];
}
void cct_oracle_saxpy(size_t n, float alpha, const float *x, float *y) {
  cct_oracle_saxpby(n, alpha, x, 1.0f, y);
}

/* ------------------------------------------------------------------------------------
 * Convolution bias.  parallel_map<_f_src_to_dst_bias_forward,_f_bias_forward>
 * (src/kernels/conv.hxx:10-26, called at src/bridges/ConvolutionBridge_impl.hxx:349-364): every
 * (batch, depth) slice of fmap floats gets bias[depth] added.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_bias_forward(float *out, const float *bias, size_t fmap, size_t depth,
                             size_t batch) {
  for (size_t sl = 0; sl < depth * batch; ++sl) {
    const float bv = bias[sl % depth];
    float *o = out + sl * fmap;
    for (size_t i = 0; i < fmap; ++i) o[i] += bv;
  }
}

/* parallel_map<_f_src_to_dst_bias_backward,_f_bias_backward> (src/kernels/conv.hxx:31-50, called
 * at src/bridges/ConvolutionBridge_impl.hxx:575-599): bias_grad is cleared, then slice sums
 * (sequential fp32) are accumulated in ascending slice order, i.e. batch-major. */
void cct_oracle_bias_backward(float *bias_grad, const float *out_grad, size_t fmap, size_t depth,
                              size_t batch) {
  for (size_t dd = 0; dd < depth; ++dd) bias_grad[dd] = 0.0f;
  for (size_t sl = 0; sl < depth * batch; ++sl) {
    const float *g = out_grad + sl * fmap;
    float sum = 0.0f;
    for (size_t i = 0; i < fmap; ++i) sum += g[i];
    bias_grad[sl % depth] += sum;
  }
}

/* ------------------------------------------------------------------------------------
 * Whole convolution, CPU branch of ConvolutionBridge.
 * forward  : src/bridges/ConvolutionBridge_impl.hxx:294-373
 * backward : src/bridges/ConvolutionBridge_impl.hxx:551-628
 * GEMM argument tuples follow Kernel::compute, src/Kernel_impl.hxx:85-170.
 * ---------------------------------------------------------------------------------- */
size_t cct_oracle_conv_m(const cct_oracle_conv_shape *c) {
  return (c->n + 2 * c->p - c->k) / c->s + 1;
}

static void conv_pmap(const cct_oracle_conv_shape *c, cct_oracle_pmap *a) {
  const size_t m = cct_oracle_conv_m(c);
  memset(a, 0, sizeof(*a));
  a->dR = c->k * c->k * c->d; a->dC = m * m * c->b; a->dD = 1; a->dB = 1;
  a->sR = c->n; a->sC = c->n; a->sD = c->d; a->sB = c->b;
  a->dBR = a->dR; a->dBC = a->dC;
  a->sBR = a->sR < 16 ? a->sR : 16; a->sBC = a->sC < 16 ? a->sC : 16;
  a->kR = c->k; a->kC = c->k; a->kD = c->d; a->kB = 1;
  a->stride = c->s; a->padding = c->p;
}

/* Connector::remap_output (src/Connector_impl_Lowering_type1.hxx:92-128): copy, then permute. */
static void remap_in_place(float *cube, size_t R, size_t C, size_t depth, size_t batch) {
  const size_t nel = R * C * depth * batch;
  float *copy = (float *)malloc(nel * sizeof(float));
  memcpy(copy, cube, nel * sizeof(float));
  cct_oracle_pmap a;
  memset(&a, 0, sizeof(a));
  a.sR = R; a.sC = C; a.sD = depth; a.sB = batch;
  a.dR = R; a.dC = C; a.dD = depth; a.dB = batch;
  cct_oracle_remap(cube, copy, &a);
  free(copy);
}

void cct_oracle_conv_forward(const cct_oracle_conv_shape *c, const float *in, const float *model,
                             const float *bias, float *lowered, float *out) {
  const size_t m = cct_oracle_conv_m(c);
  const int o = (int)c->o, kkd = (int)(c->k * c->k * c->d), bmm = (int)(c->b * m * m);
  cct_oracle_pmap a;
  conv_pmap(c, &a);
  cct_oracle_lower_cube(lowered, in, &a);
  /* KernelConfig_GEMM_NOTRANS_TRANS_NO_DIM_FLIP: out[o x b*m*m] = model[o x kkd] * lowered^T */
  cct_oracle_sgemm(CCT_ROW_MAJOR, CCT_NO_TRANS, CCT_TRANS, o, bmm, kkd, 1.0f, model, kkd, lowered,
                   kkd, 0.0f, out, bmm);
  /* [o][b][m*m] -> [b][o][m*m] */
  remap_in_place(out, m, m, c->o, c->b);
  if (bias) cct_oracle_bias_forward(out, bias, m * m, c->o, c->b);
}

void cct_oracle_conv_backward(const cct_oracle_conv_shape *c, const float *model, float *out_grad,
                              const float *lowered, float *lowered_grad, float *in_grad,
                              float *model_grad, float *bias_grad, int need_in_grad) {
  const size_t m = cct_oracle_conv_m(c);
  const int o = (int)c->o, kkd = (int)(c->k * c->k * c->d), bmm = (int)(c->b * m * m);
  if (bias_grad) cct_oracle_bias_backward(bias_grad, out_grad, m * m, c->o, c->b);
  /* [b][o][m*m] -> [o][b][m*m], in place on the caller's gradient cube */
  remap_in_place(out_grad, m, m, c->b, c->o);
  if (need_in_grad) {
    /* KernelConfig_GEMM_TRANS_NOTRANS: lowered_grad[kkd x b*m*m] = model^T * out_grad */
    cct_oracle_sgemm(CCT_ROW_MAJOR, CCT_TRANS, CCT_NO_TRANS, kkd, bmm, o, 1.0f, model, kkd,
                     out_grad, bmm, 0.0f, lowered_grad, bmm);
    memset(in_grad, 0, c->b * c->d * c->n * c->n * sizeof(float));
    cct_oracle_lift_args la;
    la.data_output_width = m; la.data_output_height = m; la.kernel_size = c->k;
    la.stride = c->s; la.padding = c->p; la.iR = c->n; la.iC = c->n; la.iD = c->d; la.iB = c->b;
    cct_oracle_inverse_lower_cube(in_grad, lowered_grad, &la);
  }
  /* KernelConfig_GEMM_NOTRANS_NOTRANS_DIM_FLIP, alpha 1 beta 0:
   * model_grad[o x kkd] = out_grad[o x b*m*m] * lowered[b*m*m x kkd] */
  cct_oracle_sgemm(CCT_ROW_MAJOR, CCT_NO_TRANS, CCT_NO_TRANS, o, kkd, bmm, 1.0f, out_grad, bmm,
                   lowered, kkd, 0.0f, model_grad, kkd);
}

/* ------------------------------------------------------------------------------------
 * SGD with momentum.  SGDGradientUpdater::update, src/algorithms/GradientUpdater.h:154-193:
 *   g += lambda*w (L2) | g += lambda*sign(w) (L1, CPUDriver::L1_update DeviceDriver_CPU.cpp:111-117)
 *   h  = stepsize*g + momentum*h
 *   w -= h
 * ---------------------------------------------------------------------------------- */
void cct_oracle_sgd_update(size_t n, float *model, float *grad, float *history, float stepsize,
                           float momentum, float lambda, int l1) {
  if (lambda != 0.0f) {
    if (l1) {
      for (size_t i = 0; i < n; ++i) grad[i] += lambda * (model[i] > 0 ? 1 : -1);
    } else {
      cct_oracle_saxpy(n, lambda, model, grad);
    }
  }
  cct_oracle_saxpby(n, stepsize, grad, momentum, history);
  cct_oracle_saxpy(n, -1.0f, history, model);
}

/* Util::get_learning_rate, src/util.h:76-93 (multistep is unsupported there as well).
 * The reference is C++ with <math.h>: pow/exp on float arguments pick the float overloads
 * (step, exp: powf; sigmoid: expf), mixed float/double arguments promote to double (inv, poly),
 * and the product with base_lr is rounded to float on return.  Pinned in
 * tests/test_learning_rate.py by float64 closed forms, schedule identities and the learning
 * rates Caffe's LeNet tutorial log prints for the inv policy. */
float cct_oracle_learning_rate(const char *policy, float base_lr, float gamma, float iter,
                               float stepsize, float power, float max_iter) {
  if (!strcmp(policy, "fixed")) return base_lr;
  if (!strcmp(policy, "step")) {
    const float step = (float)(int)(iter / stepsize);
    return base_lr * powf(gamma, step);
  }
  if (!strcmp(policy, "exp")) return base_lr * powf(gamma, iter);
  if (!strcmp(policy, "inv")) return (float)(base_lr * pow(1.0 + gamma * iter, -power));
  if (!strcmp(policy, "poly")) return (float)(base_lr * pow(1.0 - (iter / max_iter), power));
  if (!strcmp(policy, "sigmoid"))
    return (float)(base_lr * (1.0 / (1.0 + expf(-gamma * (iter - stepsize)))));
  return NAN;
}

/* ------------------------------------------------------------------------------------
 * ReLU.  src/kernels/relu.hxx:21-45 through parallel_map (ReLUBridge_impl.hxx:33-100).
 * ---------------------------------------------------------------------------------- */
void cct_oracle_relu_forward(float *out, const float *in, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = in[i] > 0.0f ? in[i] : 0.0f;
}
void cct_oracle_relu_backward(float *in_grad, const float *out_grad, const float *in_data,
                              size_t n) {
  for (size_t i = 0; i < n; ++i) in_grad[i] = out_grad[i] * (float)(in_data[i] > 0);
}

/* ------------------------------------------------------------------------------------
 * Max pooling.  CPUDriver::maxpool_forward/backward, src/sched/DeviceDriver_CPU.cpp:369-421;
 * the bridge pre-fills the output with -FLT_MAX (MaxPoolingBridge_impl.hxx:67) and clears the
 * input gradient (:123).  Strict '>' keeps the first maximum; max_index stores h*iC+w as int.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_maxpool_forward(float *out, int *max_index, const float *in, int k, int s, int iR,
                                int iC, int oR, int oC, int D, int B) {
  for (long i = 0; i < (long)D * B; ++i) {
    const float *src = in + i * iR * iC;
    float *dst = out + i * oR * oC;
    int *idx = max_index + i * oR * oC;
    for (int ph = 0; ph < oR; ++ph) {
      const int hend = ph * s + k < iR ? ph * s + k : iR;
      for (int pw = 0; pw < oC; ++pw) {
        const int wend = pw * s + k < iC ? pw * s + k : iC;
        float best = -FLT_MAX;
        int besti = idx[ph * oC + pw]; /* untouched if nothing exceeds -FLT_MAX */
        for (int h = ph * s; h < hend; ++h)
          for (int w = pw * s; w < wend; ++w)
            if (src[h * iC + w] > best) {
              best = src[h * iC + w];
              besti = h * iC + w;
            }
        dst[ph * oC + pw] = best;
        idx[ph * oC + pw] = besti;
      }
    }
  }
}

void cct_oracle_maxpool_backward(float *in_grad, const float *out_grad, const int *max_index,
                                 int iR, int iC, int oR, int oC, int D, int B) {
  memset(in_grad, 0, sizeof(float) * (size_t)iR * iC * D * B);
  for (long i = 0; i < (long)D * B; ++i)
    for (int q = 0; q < oR * oC; ++q)
      in_grad[i * iR * iC + max_index[i * oR * oC + q]] += out_grad[i * oR * oC + q];
}

/* ------------------------------------------------------------------------------------
 * Across-channel LRN.  Forward = _f_lrn_forward (running window over depth, with the same
 * copy / subtract / add order per pixel) followed by _f_lrn_forward_normalize,
 * src/kernels/lrn.hxx:46-129, driven by LRNBridge_impl.hxx:46-105.  Exact powf is used where the
 * reference's product build substitutes an approximation (lrn.hxx:11-30, Makefile:37).
 * denoms keeps 1 + alpha/size * sum(x^2) for the backward pass.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_lrn_forward(float *out, float *denoms, const float *in, int iR, int iC, int iD,
                            int iB, int local_size, float alpha, float beta) {
  const int w = local_size / 2;
  const long rc = (long)iR * iC;
  const float alpha_over_size = alpha / local_size;
  for (long ib = 0; ib < iB; ++ib) {
    const float *x = in + ib * rc * iD;
    float *dn = denoms + ib * rc * iD;
    for (long q = 0; q < rc; ++q) {
      float sum = 0.0f;
      for (int i = 0; i <= w; ++i) sum += (i >= iD) ? 0.0f : x[i * rc + q] * x[i * rc + q];
      dn[q] = sum;
    }
    for (int dd = 1; dd < iD; ++dd)
      for (long q = 0; q < rc; ++q) {
        float v = dn[(dd - 1) * rc + q];
        if (dd - w - 1 >= 0) v -= x[(dd - w - 1) * rc + q] * x[(dd - w - 1) * rc + q];
        if (dd + w < iD) v += x[(dd + w) * rc + q] * x[(dd + w) * rc + q];
        dn[dd * rc + q] = v;
      }
  }
  const long total = rc * iD * iB;
  for (long i = 0; i < total; ++i) {
    denoms[i] = alpha_over_size * denoms[i] + 1;
    out[i] = in[i] / powf(denoms[i], beta);
  }
}

/* _f_lrn_backward, src/kernels/lrn.hxx:146-179 (LRNBridge_impl.hxx:113-180 clears in_grad first).
 * Mixed float/double steps are kept as written there. */
void cct_oracle_lrn_backward(float *in_grad, const float *out_grad, const float *in_data,
                             const float *denoms, int R, int C, int D, int B, int local_size,
                             float alpha, float beta) {
  const int w = local_size / 2;
  const long rc = (long)R * C;
  const float alpha_over_size = alpha / local_size;
  memset(in_grad, 0, sizeof(float) * (size_t)rc * D * B);
  for (long ib = 0; ib < B; ++ib) {
    const long base = ib * rc * D;
    for (int od = 0; od < D; ++od)
      for (long q = 0; q < rc; ++q) {
        const float dne = denoms[base + od * rc + q];
        const float denom = powf(dne, beta);
        const float denom_n1 = (float)(1. / (denom * dne));
        const float og = out_grad[base + od * rc + q];
        const float wd = in_data[base + od * rc + q];
        const float g2 = beta * denom_n1 * alpha_over_size * 2 * wd;
        for (int i = -w; i <= w; ++i) {
          const int ch = od + i;
          if (ch < 0 || ch >= D) continue;
          const float xv = in_data[base + ch * rc + q];
          float g;
          if (i == 0) g = (float)(1. / denom - g2 * xv);
          else g = -g2 * xv;
          in_grad[base + ch * rc + q] += g * og;
        }
      }
  }
}

/* ------------------------------------------------------------------------------------
 * Dropout.  CPU flavour (mask in {0,1}): DropoutBridge_impl.hxx:68-82, 153-163.
 * Device flavour (uint32 mask, keep iff mask > threshold): src/kernels/dropout.hxx:20-32 with
 * threshold = (unsigned)(UINT_MAX * ratio), DropoutBridge_impl.hxx:35-36.
 * ---------------------------------------------------------------------------------- */
void cct_oracle_dropout_forward(float *out, const float *in, const unsigned int *mask, float ratio,
                                size_t n) {
  const float scale = (float)(1. / (1. - ratio));
  for (size_t i = 0; i < n; ++i) out[i] = in[i] * mask[i] * scale;
}
void cct_oracle_dropout_forward_threshold(float *out, const float *in, const unsigned int *mask,
                                          float ratio, size_t n) {
  const float scale = (float)(1. / (1. - ratio));
  const unsigned int thr = (unsigned int)(4294967295u * ratio);
  for (size_t i = 0; i < n; ++i) out[i] = in[i] * (mask[i] > thr) * scale;
}

/* ------------------------------------------------------------------------------------
 * Softmax with multinomial logistic loss.  src/kernels/softmax.hxx:19-81 driven by
 * SoftmaxLossBridge_impl.hxx:36-143.  Labels are floats, one per image.  Returns the summed
 * loss over the batch (the caller divides by the batch size, src/DeepNet.h:2139).
 * ---------------------------------------------------------------------------------- */
float cct_oracle_softmax_loss_forward(float *prob, const float *in, const float *labels, size_t iR,
                                      size_t iC, size_t iD, size_t iB) {
  const size_t len = iR * iC * iD;
  float loss = 0.0f;
  for (size_t ib = 0; ib < iB; ++ib) {
    const float *x = in + ib * len;
    float *y = prob + ib * len;
    float mx = x[0];
    for (size_t i = 1; i < len; ++i)
      if (x[i] > mx) mx = x[i];
    float denom = 0.0f;
    for (size_t i = 0; i < len; ++i) denom += expf(x[i] - mx);
    for (size_t i = 0; i < len; ++i) y[i] = expf(x[i] - mx) / denom;
    const float pl = y[(int)labels[ib]];
    loss -= logf(pl > FLT_MIN ? pl : FLT_MIN);
  }
  return loss;
}

void cct_oracle_softmax_loss_backward(float *in_grad, const float *prob, const float *labels,
                                      size_t iR, size_t iC, size_t iD, size_t iB) {
  const size_t len = iR * iC * iD;
  memcpy(in_grad, prob, len * iB * sizeof(float));
  for (size_t ib = 0; ib < iB; ++ib) {
    float *g = in_grad + ib * len;
    g[(int)labels[ib]] -= 1;
    for (size_t i = 0; i < len; ++i) g[i] = (float)(g[i] * (1. / iB / (iR * iC)));
  }
}

/* ------------------------------------------------------------------------------------
 * Fully connected layer through sgemm_new.  FullyConnectedBridge_impl.hxx:169-234 (forward:
 * Y = X * W^T, bias added by a rank-1 GEMM with a ones vector) and :255-326 (backward: bias
 * gradient by gemv with ones, dX = dY * W, dW = dY^T * X).
 * ---------------------------------------------------------------------------------- */
void cct_oracle_fc_forward(float *out, const float *in, const float *model, const float *bias,
                           int B, int I, int O) {
  cct_oracle_sgemm_new(CCT_NO_TRANS, CCT_TRANS, B, O, I, 1.0f, in, model, 0.0f, out);
  if (bias) {
    float *ones = (float *)malloc(sizeof(float) * (size_t)B);
    for (int i = 0; i < B; ++i) ones[i] = 1.0f;
    cct_oracle_sgemm_new(CCT_NO_TRANS, CCT_NO_TRANS, B, O, 1, 1.0f, ones, bias, 1.0f, out);
    free(ones);
  }
}

void cct_oracle_fc_backward(float *in_grad, float *model_grad, float *bias_grad, const float *in,
                            const float *model, const float *out_grad, int B, int I, int O,
                            int need_in_grad) {
  if (bias_grad) {
    float *ones = (float *)malloc(sizeof(float) * (size_t)B);
    for (int i = 0; i < B; ++i) ones[i] = 1.0f;
    cct_oracle_sgemv(CCT_TRANS, B, O, 1.0f, out_grad, ones, 0.0f, bias_grad);
    free(ones);
  }
  if (need_in_grad)
    cct_oracle_sgemm_new(CCT_NO_TRANS, CCT_NO_TRANS, B, I, O, 1.0f, out_grad, model, 0.0f, in_grad);
  cct_oracle_sgemm_new(CCT_TRANS, CCT_NO_TRANS, O, I, B, 1.0f, out_grad, in, 0.0f, model_grad);
}

/* ------------------------------------------------------------------------------------
 * One image through the input transform.  Restates Corpus::process_image
 * (src/parser/corpus.h:262-333) for byte data: with a crop, the window starting at
 * (h_off, w_off) is copied, columns reversed when `mirror` is set; element =
 * (float(byte) - mean[same source index]) * scale.  Without a crop the whole image is converted.
 * The caller supplies h_off / w_off / mirror (the reference draws them with rand()).
 * ---------------------------------------------------------------------------------- */
void cct_oracle_process_image(float *out, const unsigned char *data, const float *mean, int channels,
                              int height, int width, int crop_size, int h_off, int w_off, int mirror,
                              float scale) {
  if (crop_size > 0) {
    for (int c = 0; c < channels; ++c)
      for (int h = 0; h < crop_size; ++h)
        for (int w = 0; w < crop_size; ++w) {
          const int data_index = (c * height + h + h_off) * width + w + w_off;
          const int top_index = mirror ? (c * crop_size + h) * crop_size + (crop_size - 1 - w)
                                       : (c * crop_size + h) * crop_size + w;
          const float e = (float)data[data_index];
          out[top_index] = (e - (mean ? mean[data_index] : 0.0f)) * scale;
        }
  } else {
    const long n = (long)channels * height * width;
    for (long i = 0; i < n; ++i) out[i] = ((float)data[i] - (mean ? mean[i] : 0.0f)) * scale;
  }
}
