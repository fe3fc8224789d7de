// Inner-product layers with a handful of outputs (LeNet's last layer: 500 -> 10 at batch 64).
//
//   forward   Y[B x O]  = X[B x I] * W[O x I]^T + bias          (+ clamp of a following in-place ReLU)
//   backward  dX[B x I] = dY[B x O] * W                         (masked by the ReLU before the layer, if told)
//             dW[O x I] = dY^T * X,   db[O] = column sums of dY
//
// These are the three sgemm_new calls and the bias passes of FullyConnectedBridge
// (src/bridges/FullyConnectedBridge_impl.hxx:169-234, 255-326).  With O of a few dozen at most, a 64 x 64
// MFMA tile is nearly all padding and the layer is a handful of launches of 2-10 us each (GEMM, split-K
// reduction, bias, ReLU mask); here the forward pass is ONE launch and the backward pass is ONE launch of
// plain fp32 FMAs -- the arithmetic is a few hundred kFLOP, the time is launch latency.  HBM-bound in
// principle (every operand is read once), latency-bound in practice.
//
// Summation orders are fixed (no atomics): run-to-run identical results.
#include "cct_common.h"

namespace cct {

constexpr int FCS_THREADS = 256;
constexpr int kFcSmallMaxOut = 32;
constexpr int kFcSmallMaxBatch = 1024;

__device__ __forceinline__ float fcs_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// One workgroup per image: lane t takes inputs t, t + 256, ... against all O rows of W (consecutive lanes read
// consecutive words of X and of every row of W), then the O partial sums are added over the wavefront (shuffle
// tree) and over the four wavefronts in order.
template <int OMAX>
__global__ __launch_bounds__(FCS_THREADS) void fc_small_forward_kernel(float *__restrict__ y,
                                                                      const float *__restrict__ x,
                                                                      const float *__restrict__ w,
                                                                      const float *__restrict__ bias, int in, int out,
                                                                      int relu) {
  __shared__ float part[FCS_THREADS / 64][OMAX];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float *xb = x + (size_t)b * in;
  float acc[OMAX];
#pragma unroll
  for (int n = 0; n < OMAX; ++n) acc[n] = 0.0f;
  // two strides of the input per trip: all of their loads are issued before the first multiply-add, so a layer of up
  // to 512 inputs pays one memory latency, not one per stride (k ascending within a lane either way)
  for (int k0 = tid; k0 < in; k0 += 2 * FCS_THREADS) {
    const int k1 = k0 + FCS_THREADS;
    const bool two = k1 < in;
    const float x0 = xb[k0], x1 = two ? xb[k1] : 0.0f;
    float w0[OMAX], w1[OMAX];
#pragma unroll
    for (int n = 0; n < OMAX; ++n) {
      w0[n] = n < out ? w[(size_t)n * in + k0] : 0.0f;
      w1[n] = (n < out && two) ? w[(size_t)n * in + k1] : 0.0f;
    }
#pragma unroll
    for (int n = 0; n < OMAX; ++n) acc[n] += x0 * w0[n];
#pragma unroll
    for (int n = 0; n < OMAX; ++n) acc[n] += x1 * w1[n];
  }
#pragma unroll
  for (int n = 0; n < OMAX; ++n) {
    const float s = fcs_wave_sum(acc[n]);
    if ((tid & 63) == 0) part[tid >> 6][n] = s;
  }
  __syncthreads();
  if (tid < out) {
    float s = part[0][tid];
#pragma unroll
    for (int wv = 1; wv < FCS_THREADS / 64; ++wv) s += part[wv][tid];
    if (bias) s += bias[tid];
    y[(size_t)b * out + tid] = (relu && !(s > 0.0f)) ? 0.0f : s;
  }
}

// One launch for the whole backward pass.  Workgroups [0, nb_dx): one lane per element of dX (O multiply-adds;
// consecutive lanes read consecutive words of every row of W).  Workgroups [nb_dx, nb_dx + nb_dw): one lane per
// element of dW, summing over the batch in ascending image order (consecutive lanes read consecutive words of
// every row of X).  The last workgroup: lane n < O sums column n of dY.
__global__ __launch_bounds__(FCS_THREADS) void fc_small_backward_kernel(float *__restrict__ dx, float *__restrict__ dw,
                                                                       float *__restrict__ db,
                                                                       const float *__restrict__ dy,
                                                                       const float *__restrict__ x,
                                                                       const float *__restrict__ w,
                                                                       const float *__restrict__ relu_data, int batch,
                                                                       int in, int out, uint32_t nb_dx, uint32_t nb_dw,
                                                                       FastDiv div_in) {
  const uint32_t blk = blockIdx.x, tid = threadIdx.x;
  if (blk < nb_dx) {
    const uint32_t e = blk * FCS_THREADS + tid;
    if (e >= (uint32_t)batch * in) return;
    const uint32_t b = fdiv(e, div_in), k = e - b * in;
    const float *g = dy + (size_t)b * out;
    float s = 0.0f;
    int n = 0;
    for (; n + 8 <= out; n += 8) {   // eight rows of W in flight per lane, added in row order
      float wv[8], gv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        wv[j] = w[(size_t)(n + j) * in + k];
        gv[j] = g[n + j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) s += gv[j] * wv[j];
    }
    for (; n < out; ++n) s += g[n] * w[(size_t)n * in + k];
    if (relu_data && !(relu_data[e] > 0.0f)) s = 0.0f;
    dx[e] = s;
  } else if (blk < nb_dx + nb_dw) {
    const uint32_t e = (blk - nb_dx) * FCS_THREADS + tid;
    if (e >= (uint32_t)out * in) return;
    const uint32_t n = fdiv(e, div_in), k = e - n * in;
    float s = 0.0f;
    int b = 0;
    // sixteen images in flight per lane (the loop is bound by memory latency), added in image order
    for (; b + 16 <= batch; b += 16) {
      float xv[16], gv[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        xv[j] = x[(size_t)(b + j) * in + k];
        gv[j] = dy[(size_t)(b + j) * out + n];
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) s += gv[j] * xv[j];
    }
    for (; b < batch; ++b) s += dy[(size_t)b * out + n] * x[(size_t)b * in + k];
    dw[e] = s;
  } else if (db && tid < (uint32_t)out) {
    float s = 0.0f;
    for (int b = 0; b < batch; ++b) s += dy[(size_t)b * out + tid];
    db[tid] = s;
  }
}

static bool fc_small_covers(int batch, int in, int out) {
  return batch > 0 && in > 0 && out > 0 && out <= kFcSmallMaxOut && batch <= kFcSmallMaxBatch &&
         (double)batch * in < 1073741824.0 && (double)out * in < 1073741824.0;
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_fc_small_supported(int batch, int in_features, int out_features) {
  return fc_small_covers(batch, in_features, out_features) ? 1 : 0;
}

extern "C" int cct_hip_fc_small_forward(float *y, const float *x, const float *w, const float *bias, int batch,
                                        int in_features, int out_features, int relu) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(y && x && w, "fc_small_forward: null argument");
  CCT_REQUIRE(fc_small_covers(batch, in_features, out_features),
              "fc_small_forward: sizes not covered (batch %d, %d -> %d)", batch, in_features, out_features);
  if (out_features <= 16)
    hipLaunchKernelGGL(fc_small_forward_kernel<16>, dim3(batch), dim3(FCS_THREADS), 0, ctx().stream, y, x, w, bias,
                       in_features, out_features, relu);
  else
    hipLaunchKernelGGL(fc_small_forward_kernel<kFcSmallMaxOut>, dim3(batch), dim3(FCS_THREADS), 0, ctx().stream, y, x,
                       w, bias, in_features, out_features, relu);
  CCT_LAUNCH_CHECK();
  note_kernel("fc_small_forward_kernel<%d>", out_features <= 16 ? 16 : kFcSmallMaxOut);
  return 0;
}

extern "C" int cct_hip_fc_small_backward(float *dx, float *dw, float *db, const float *dy, const float *x,
                                         const float *w, int batch, int in_features, int out_features,
                                         const float *relu_data) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dw && dy && x && w, "fc_small_backward: null argument");
  CCT_REQUIRE(dx || !relu_data, "fc_small_backward: a ReLU mask without an input gradient to mask");
  CCT_REQUIRE(fc_small_covers(batch, in_features, out_features),
              "fc_small_backward: sizes not covered (batch %d, %d -> %d)", batch, in_features, out_features);
  const uint32_t nb_dx = dx ? (uint32_t)(((size_t)batch * in_features + FCS_THREADS - 1) / FCS_THREADS) : 0u;
  const uint32_t nb_dw = (uint32_t)(((size_t)out_features * in_features + FCS_THREADS - 1) / FCS_THREADS);
  hipLaunchKernelGGL(fc_small_backward_kernel, dim3(nb_dx + nb_dw + 1), dim3(FCS_THREADS), 0, ctx().stream, dx, dw, db,
                     dy, x, w, relu_data, batch, in_features, out_features, nb_dx, nb_dw,
                     make_fastdiv((uint32_t)in_features));
  CCT_LAUNCH_CHECK();
  note_kernel("fc_small_backward_kernel");
  return 0;
}
