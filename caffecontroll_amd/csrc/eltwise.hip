// HBM-bound helper kernels of the driver: slice remap, bias add, ReLU, max pooling, LRN, dropout,
// softmax loss, BLAS-1 / SGD update, fills and gemv.  One pass over the data each; 16-byte
// vector accesses where the element count and alignment allow it.
#include <cfloat>
#include <cstring>

#include "cct_common.h"
#include "colsum.h"

namespace cct {

constexpr int TPB = 256;

static inline uint32_t blocks_for(size_t n, int per_block = TPB) {
  return (uint32_t)((n + per_block - 1) / per_block);
}

__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off, 64));
  return v;
}

// Reduction of one value per lane over a 256-lane workgroup; result valid on every lane.
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float *scratch /* >= 5 floats */) {
  v = MAX ? wave_max_f(v) : wave_sum_f(v);
  const int tid = threadIdx.x;
  __syncthreads();
  if ((tid & 63) == 0) scratch[tid >> 6] = v;
  __syncthreads();
  if (tid == 0) {
    float t = scratch[0];
    for (int w = 1; w < TPB / 64; ++w) t = MAX ? fmaxf(t, scratch[w]) : t + scratch[w];
    scratch[4] = t;
  }
  __syncthreads();
  return scratch[4];
}

// ---- fills --------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void fill_f32_kernel(float *__restrict__ p, size_t n, float v) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) p[i] = v;
}
__global__ __launch_bounds__(TPB) void fill_u8_kernel(unsigned char *__restrict__ p, size_t n,
                                                      unsigned char v) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) p[i] = v;
}

// ---- slice remap: dst slice (j / sB) + (j % sB) * sD  <-  src slice j --------------------------
// A workgroup moves one slice (or, for long slices, one of gridDim.y parts of it) with 16-byte loads
// and stores at dword alignment, four of them in flight per lane.
typedef float remap_f4u __attribute__((ext_vector_type(4), aligned(4)));

__global__ __launch_bounds__(TPB) void remap_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                    uint32_t rc, uint32_t sD, FastDiv div_b) {
  const uint32_t j = blockIdx.x;  // source slice
  const uint32_t reald = fdiv(j, div_b);
  const uint32_t realb = j - reald * div_b.div;
  const float *s = src + (size_t)j * rc;
  float *d = dst + ((size_t)reald + (size_t)realb * sD) * rc;
  const uint32_t nq = rc >> 2, stride = gridDim.y * TPB;
  for (uint32_t q0 = blockIdx.y * TPB + threadIdx.x; q0 < nq; q0 += 4 * stride) {
    remap_f4u v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (q0 + u * stride < nq) v[u] = *reinterpret_cast<const remap_f4u *>(s + 4 * (size_t)(q0 + u * stride));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (q0 + u * stride < nq) *reinterpret_cast<remap_f4u *>(d + 4 * (size_t)(q0 + u * stride)) = v[u];
  }
  if (blockIdx.y == 0 && threadIdx.x < (rc & 3u)) d[4 * nq + threadIdx.x] = s[4 * nq + threadIdx.x];
}

// The same copy for the backward pass of a convolution that also wants its bias gradient: source
// slice j = (image j / sB, map j % sB); while a workgroup moves its part of a slice it adds up
// what it moves (lanes in a fixed pattern, then a workgroup reduction) and leaves the sum in
// partial[j * gridDim.y + part].  bias_partial_sum_kernel adds those per map in a fixed order.
__global__ __launch_bounds__(TPB) void remap_bias_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                         uint32_t rc, uint32_t sD, FastDiv div_b,
                                                         float *__restrict__ partial) {
  __shared__ float red[8];
  const uint32_t j = blockIdx.x;  // source slice
  const uint32_t reald = fdiv(j, div_b);
  const uint32_t realb = j - reald * div_b.div;
  const float *s = src + (size_t)j * rc;
  float *d = dst + ((size_t)reald + (size_t)realb * sD) * rc;
  const uint32_t nq = rc >> 2, stride = gridDim.y * TPB;
  float sum = 0.0f;
  for (uint32_t q0 = blockIdx.y * TPB + threadIdx.x; q0 < nq; q0 += 4 * stride) {
    remap_f4u v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (q0 + u * stride < nq) v[u] = *reinterpret_cast<const remap_f4u *>(s + 4 * (size_t)(q0 + u * stride));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (q0 + u * stride < nq) {
        *reinterpret_cast<remap_f4u *>(d + 4 * (size_t)(q0 + u * stride)) = v[u];
        sum += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
      }
  }
  if (blockIdx.y == 0 && threadIdx.x < (rc & 3u)) {
    const float t = s[4 * nq + threadIdx.x];
    d[4 * nq + threadIdx.x] = t;
    sum += t;
  }
  sum = block_reduce<false>(sum, red);
  if (threadIdx.x == 0) partial[(size_t)j * gridDim.y + blockIdx.y] = sum;
}

// bias[o] = sum over images b and parts of partial[(b * O + o) * parts + part]; one workgroup per map
__global__ __launch_bounds__(TPB) void bias_partial_sum_kernel(float *__restrict__ bias, const float *__restrict__ partial,
                                                               uint32_t O, uint32_t B, uint32_t parts) {
  __shared__ float red[8];
  const uint32_t o = blockIdx.x;
  float sum = 0.0f;
  for (uint32_t i = threadIdx.x; i < B * parts; i += TPB) {
    const uint32_t b = i / parts, part = i - b * parts;
    sum += partial[((size_t)b * O + o) * parts + part];
  }
  sum = block_reduce<false>(sum, red);
  if (threadIdx.x == 0) bias[o] = sum;
}

// ---- depth-slice copy: part [B][dc][rc] <-> channels [d_off, d_off+dc) of whole [B][D][rc] ----------
__global__ __launch_bounds__(TPB) void depth_slice_kernel(float *__restrict__ part, float *__restrict__ whole,
                                                          uint32_t per_image, uint32_t whole_stride,
                                                          uint32_t whole_off, int gather) {
  const uint32_t b = blockIdx.y;
  float *p = part + (size_t)b * per_image;
  float *w = whole + (size_t)b * whole_stride + whole_off;
  for (uint32_t i = blockIdx.x * TPB + threadIdx.x; i < per_image; i += gridDim.x * TPB) {
    if (gather) p[i] = w[i];
    else w[i] = p[i];
  }
}

// ---- bias forward: out[slice][i] += bias[slice % depth] ----------------------------------------
__global__ __launch_bounds__(TPB) void bias_forward_kernel(float *__restrict__ out,
                                                           const float *__restrict__ bias, uint32_t fmap,
                                                           FastDiv div_depth) {
  const uint32_t sl = blockIdx.x;
  const uint32_t q = fdiv(sl, div_depth);
  const float bv = bias[sl - q * div_depth.div];
  float *o = out + (size_t)sl * fmap;
  for (uint32_t i = blockIdx.y * TPB + threadIdx.x; i < fmap; i += gridDim.y * TPB) o[i] += bv;
}

// small feature maps (FC layers have fmap = 1): one lane per element
__global__ __launch_bounds__(TPB) void bias_forward_flat_kernel(float *__restrict__ out,
                                                                const float *__restrict__ bias, uint32_t total,
                                                                FastDiv div_fmap, FastDiv div_depth) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  const uint32_t sl = fdiv(e, div_fmap);
  const uint32_t q = fdiv(sl, div_depth);
  out[e] += bias[sl - q * div_depth.div];
}

// ---- FC bias gradient: bias[d] = sum_b out[b][d] ------------------------------------------------
// A workgroup owns 64 columns; its four wavefronts sum a quarter of the rows each, eight loads in
// flight per lane, and the four partial sums are added in a fixed order.
__global__ __launch_bounds__(TPB) void bias_backward_fc_kernel(float *__restrict__ bias,
                                                               const float *__restrict__ og, int D, int B) {
  __shared__ float part[4][64];
  colsum_block(bias, og, D, B, blockIdx.x, part);
}

// ---- ReLU ----------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void relu_fwd_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                       size_t n) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) {
    const float x = in[i];
    out[i] = x > 0.0f ? x : 0.0f;
  }
}
__global__ __launch_bounds__(TPB) void relu_bwd_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                       const float *__restrict__ x, size_t n) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride)
    ig[i] = og[i] * (x[i] > 0.0f ? 1.0f : 0.0f);
}

// ---- max pooling -----------------------------------------------------------------------------
// forward: one lane per output element; window scanned row-major with strict '>' so that the
// first maximum wins, index stored as h*iC + w (int), as CPUDriver::maxpool_forward does
__global__ __launch_bounds__(TPB) void maxpool_fwd_kernel(float *__restrict__ out, int *__restrict__ idx,
                                                          const float *__restrict__ in, cct_pool_args a,
                                                          uint32_t total, FastDiv div_oc, FastDiv div_or) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  const uint32_t t1 = fdiv(e, div_oc);
  const int pw = e - t1 * a.oC;
  const uint32_t plane = fdiv(t1, div_or);
  const int ph = t1 - plane * a.oR;
  const float *src = in + (size_t)plane * a.iR * a.iC;
  const int h0 = ph * a.stride, w0 = pw * a.stride;
  const int h1 = min(h0 + a.kernel_size, a.iR), w1 = min(w0 + a.kernel_size, a.iC);
  float best = -FLT_MAX;
  int besti = 0;
  for (int h = h0; h < h1; ++h)
    for (int w = w0; w < w1; ++w) {
      const float v = src[h * a.iC + w];
      if (v > best) {
        best = v;
        besti = h * a.iC + w;
      }
    }
  out[e] = best;
  idx[e] = besti;
}

// backward as a gather: one lane per input element sums the output gradients whose argmax is this
// element, scanning candidate windows in (ph, pw) ascending order = the order of the
// reference's scatter loop, so sums with several contributors are bit-identical
template <bool TWO_BY_TWO>
__global__ __launch_bounds__(TPB) void maxpool_bwd_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                          const int *__restrict__ idx, cct_pool_args a,
                                                          uint32_t total, FastDiv div_ic, FastDiv div_ir) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  const uint32_t t1 = fdiv(e, div_ic);
  const int w = e - t1 * a.iC;
  const uint32_t plane = fdiv(t1, div_ir);
  const int h = t1 - plane * a.iR;
  const int k = a.kernel_size, s = a.stride;
  const int ph_lo = h < k ? 0 : (h - k) / s + 1, ph_hi = min(h / s, a.oR - 1);
  const int pw_lo = w < k ? 0 : (w - k) / s + 1, pw_hi = min(w / s, a.oC - 1);
  const int me = h * a.iC + w;
  const size_t obase = (size_t)plane * a.oR * a.oC;
  float acc = 0.0f;
  if (TWO_BY_TWO) {
    // kernel <= 2*stride: an element lies in at most two windows per direction.  All candidates are
    // fetched at once (clamped positions, so the loads need no branches) and added in (ph, pw) order.
    int cidx[2][2];
    float cog[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const size_t o = obase + min(ph_lo + i, a.oR - 1) * a.oC + min(pw_lo + j, a.oC - 1);
        cidx[i][j] = idx[o];
        cog[i][j] = og[o];
      }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (ph_lo + i <= ph_hi && pw_lo + j <= pw_hi && cidx[i][j] == me) acc += cog[i][j];
  } else {
    for (int ph = ph_lo; ph <= ph_hi; ++ph)
      for (int pw = pw_lo; pw <= pw_hi; ++pw) {
        const size_t o = obase + ph * a.oC + pw;
        if (idx[o] == me) acc += og[o];
      }
  }
  ig[e] = acc;
}

// Plane-tiled variants: a workgroup owns `pp` consecutive (image, channel) planes, brings what the
// gathers read into LDS with contiguous 16-byte loads (forward: the input planes; backward: the
// output gradient and argmax planes; several loads in flight per lane) and writes contiguous
// results, so HBM sees every byte once and the strided / repeated accesses hit LDS.  Same scan
// orders as the kernels above, hence the same bits.
constexpr int kPoolLdsWords = 8192;  // 32 KB
typedef float pool_f4u __attribute__((ext_vector_type(4), aligned(4)));
typedef int pool_i4u __attribute__((ext_vector_type(4), aligned(4)));

// dst[0..n) (LDS) = src[0..n) (global, 4-byte aligned): 16-byte loads, UNR of them in flight per lane
template <typename V4, typename T, int UNR>
__device__ __forceinline__ void pool_stage(T *dst, const T *__restrict__ src, uint32_t n) {
  const uint32_t n4 = n >> 2;
  for (uint32_t base = 0; base < n4; base += TPB * UNR) {
    V4 v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const uint32_t q = base + u * TPB + threadIdx.x;
      if (q < n4) v[u] = *reinterpret_cast<const V4 *>(src + 4 * q);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const uint32_t q = base + u * TPB + threadIdx.x;
      if (q < n4) {
        dst[4 * q] = v[u][0]; dst[4 * q + 1] = v[u][1]; dst[4 * q + 2] = v[u][2]; dst[4 * q + 3] = v[u][3];
      }
    }
  }
  if (threadIdx.x < (n & 3u)) dst[4 * n4 + threadIdx.x] = src[4 * n4 + threadIdx.x];
}

// dst[i] (LDS) = y[i] > 0 ? g[i] : 0 for i in [0, n): the output gradient of a pooling layer with
// the windows whose maximum is not positive switched off (both global arrays 4-byte aligned)
template <int UNR>
__device__ __forceinline__ void pool_stage_masked(float *dst, const float *__restrict__ g,
                                                  const float *__restrict__ y, uint32_t n) {
  const uint32_t n4 = n >> 2;
  for (uint32_t base = 0; base < n4; base += TPB * UNR) {
    pool_f4u gv[UNR], yv[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const uint32_t q = base + u * TPB + threadIdx.x;
      if (q < n4) {
        gv[u] = *reinterpret_cast<const pool_f4u *>(g + 4 * q);
        yv[u] = *reinterpret_cast<const pool_f4u *>(y + 4 * q);
      }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const uint32_t q = base + u * TPB + threadIdx.x;
      if (q < n4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[4 * q + e] = yv[u][e] > 0.0f ? gv[u][e] : 0.0f;
      }
    }
  }
  if (threadIdx.x < (n & 3u)) {
    const uint32_t i = 4 * n4 + threadIdx.x;
    dst[i] = y[i] > 0.0f ? g[i] : 0.0f;
  }
}

// out[i] = y[i] > 0 ? g[i] : 0 in global memory (the same switch for the kernels that do not stage)
__global__ __launch_bounds__(TPB) void mask_positive_kernel(float *__restrict__ out, const float *__restrict__ g,
                                                            const float *__restrict__ y, size_t n) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) out[i] = y[i] > 0.0f ? g[i] : 0.0f;
}

__global__ __launch_bounds__(TPB) void maxpool_fwd_plane_kernel(float *__restrict__ out, int *__restrict__ idx,
                                                                const float *__restrict__ in, cct_pool_args a,
                                                                uint32_t planes, int pp, FastDiv div_oc,
                                                                FastDiv div_oplane) {
  extern __shared__ float pool_lds[];  // pp * iplane words, sized by the launch
  float *tile = pool_lds;
  const uint32_t p0 = blockIdx.x * (uint32_t)pp;
  const uint32_t np = min((uint32_t)pp, planes - p0);
  const uint32_t iplane = (uint32_t)(a.iR * a.iC), oplane = (uint32_t)(a.oR * a.oC);
  pool_stage<pool_f4u, float, 8>(tile, in + (size_t)p0 * iplane, np * iplane);
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < np * oplane; i += TPB) {
    const uint32_t pl = fdiv(i, div_oplane), e = i - pl * oplane;
    const int ph = (int)fdiv(e, div_oc), pw = (int)e - ph * a.oC;
    const float *t = tile + pl * iplane;
    const int h0 = ph * a.stride, w0 = pw * a.stride;
    const int h1 = min(h0 + a.kernel_size, a.iR), w1 = min(w0 + a.kernel_size, a.iC);
    float best = -FLT_MAX;
    int besti = 0;
    for (int h = h0; h < h1; ++h)
      for (int w = w0; w < w1; ++w) {
        const float v = t[h * a.iC + w];
        if (v > best) {
          best = v;
          besti = h * a.iC + w;
        }
      }
    out[(size_t)p0 * oplane + i] = best;
    idx[(size_t)p0 * oplane + i] = besti;
  }
}

template <bool TWO_BY_TWO>
__global__ __launch_bounds__(TPB) void maxpool_bwd_plane_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                                const int *__restrict__ idx, cct_pool_args a,
                                                                uint32_t planes, int pp, FastDiv div_ic,
                                                                FastDiv div_iplane, FastDiv div_s) {
  __shared__ float tog[kPoolLdsWords / 2];
  __shared__ int tidx[kPoolLdsWords / 2];
  const uint32_t p0 = blockIdx.x * (uint32_t)pp;
  const uint32_t np = min((uint32_t)pp, planes - p0);
  const uint32_t iplane = (uint32_t)(a.iR * a.iC), oplane = (uint32_t)(a.oR * a.oC);
  pool_stage<pool_f4u, float, 4>(tog, og + (size_t)p0 * oplane, np * oplane);
  pool_stage<pool_i4u, int, 4>(tidx, idx + (size_t)p0 * oplane, np * oplane);
  __syncthreads();
  const int k = a.kernel_size;
  for (uint32_t i = threadIdx.x; i < np * iplane; i += TPB) {
    const uint32_t pl = fdiv(i, div_iplane), me = i - pl * iplane;
    const int h = (int)fdiv(me, div_ic), w = (int)me - h * a.iC;
    const int ph_lo = h < k ? 0 : (int)fdiv((uint32_t)(h - k), div_s) + 1, ph_hi = min((int)fdiv((uint32_t)h, div_s), a.oR - 1);
    const int pw_lo = w < k ? 0 : (int)fdiv((uint32_t)(w - k), div_s) + 1, pw_hi = min((int)fdiv((uint32_t)w, div_s), a.oC - 1);
    const float *g = tog + pl * oplane;
    const int *x = tidx + pl * oplane;
    float acc = 0.0f;
    if (TWO_BY_TWO) {
      // kernel <= 2*stride: at most two windows per direction; clamped positions keep the reads branch-free
      const int r0 = min(ph_lo, a.oR - 1) * a.oC, r1 = min(ph_lo + 1, a.oR - 1) * a.oC;
      const int c0 = min(pw_lo, a.oC - 1), c1 = min(pw_lo + 1, a.oC - 1);
      const int x00 = x[r0 + c0], x01 = x[r0 + c1], x10 = x[r1 + c0], x11 = x[r1 + c1];
      const float g00 = g[r0 + c0], g01 = g[r0 + c1], g10 = g[r1 + c0], g11 = g[r1 + c1];
      const bool row1 = ph_lo + 1 <= ph_hi, col1 = pw_lo + 1 <= pw_hi, any = ph_lo <= ph_hi && pw_lo <= pw_hi;
      if (any && x00 == (int)me) acc += g00;
      if (any && col1 && x01 == (int)me) acc += g01;
      if (any && row1 && x10 == (int)me) acc += g10;
      if (any && row1 && col1 && x11 == (int)me) acc += g11;
    } else {
      for (int ph = ph_lo; ph <= ph_hi; ++ph)
        for (int pw = pw_lo; pw <= pw_hi; ++pw)
          if (x[ph * a.oC + pw] == (int)me) acc += g[ph * a.oC + pw];
    }
    ig[(size_t)p0 * iplane + i] = acc;
  }
}

// The same for 2 <= stride, kernel <= 2*stride and rows of at most 256 elements, four consecutive
// elements of a row per lane: `lpr` lanes per row (the power of two >= ceil(iC / 4)), 64 / lpr rows
// per wavefront and pass.  The windows that can hold any of the four elements lie in two window
// rows and at most four window columns; the lane reads those eight (argmax, gradient) pairs once
// and tests each against its four positions -- an argmax equals a position only if the window
// contains it, so no range logic is needed beyond masking the clamped duplicates at the borders.
// Additions stay in (ph, pw) order.  One 16-byte store per lane instead of four 4-byte ones, and
// a quarter of the LDS reads and index arithmetic of the element-wise kernel.
// K3S2 = true: 3 x 3 windows with stride 2 (the CaffeNet pooling layers).  Columns w0..w0+3 (w0 a multiple of 4)
// can only lie in window columns c-1, c, c+1 with c = w0/2 -- w0 in c-1 and c, w0+1 in c, w0+2 in c and c+1,
// w0+3 in c+1 -- so six (argmax, gradient) pairs are read and twelve tests made instead of eight and thirty-two.
template <bool K3S2>
__global__ __launch_bounds__(TPB) void maxpool_bwd_quad_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                               const int *__restrict__ idx, cct_pool_args a,
                                                               uint32_t planes, int pp, int lpr_shift, FastDiv div_ir,
                                                               FastDiv div_s, const float *__restrict__ relu_data,
                                                               const float *__restrict__ pooled) {
  // relu_data (optional): the pooled tensor itself when it is the output of an in-place ReLU; the
  // gradient is then stored already masked with (relu_data > 0), which is that ReLU's backward.
  // pooled (optional, instead of relu_data): the pooling OUTPUT.  A gradient lands only on a
  // window's arg-max, whose activation is the window's maximum, so masking every window's gradient
  // with (pooled > 0) while it is staged gives the same sums and reads a tensor a quarter the size.
  // LDS sized by the launch (2 * pp * oplane words): small planes leave room for more workgroups
  // per compute unit, whose load and store phases then overlap
  extern __shared__ float pool_lds[];
  const uint32_t p0 = blockIdx.x * (uint32_t)pp;
  const uint32_t np = min((uint32_t)pp, planes - p0);
  const uint32_t iplane = (uint32_t)(a.iR * a.iC), oplane = (uint32_t)(a.oR * a.oC);
  float *tog = pool_lds;
  int *tidx = reinterpret_cast<int *>(pool_lds + (size_t)pp * oplane);
  if (pooled) pool_stage_masked<4>(tog, og + (size_t)p0 * oplane, pooled + (size_t)p0 * oplane, np * oplane);
  else pool_stage<pool_f4u, float, 4>(tog, og + (size_t)p0 * oplane, np * oplane);
  pool_stage<pool_i4u, int, 4>(tidx, idx + (size_t)p0 * oplane, np * oplane);
  __syncthreads();
  const int k = a.kernel_size;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int w0 = 4 * (lane & ((1 << lpr_shift) - 1)), rows_per_wave = 64 >> lpr_shift;
  if (w0 >= a.iC) return;
  const int nw = min(4, a.iC - w0);  // elements of this lane's quad inside the row
  // window columns pc0 .. pc0+3 (clamped; cv[j] false for the duplicates the clamp makes)
  const int pc0 = K3S2 ? (w0 >> 1) - 1 : w0 < k ? 0 : (int)fdiv((uint32_t)(w0 - k), div_s) + 1;
  constexpr int NJ = K3S2 ? 3 : 4;
  int pc[NJ];
  bool cv[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    pc[j] = min(max(pc0 + j, 0), a.oC - 1);
    cv[j] = pc0 + j >= 0 && pc0 + j <= a.oC - 1;
  }
  float *dst = ig + (size_t)p0 * iplane + w0;
  const uint32_t nrows = np * (uint32_t)a.iR;
  for (uint32_t row = wave * rows_per_wave + (lane >> lpr_shift); row < nrows; row += (TPB / 64) * rows_per_wave) {
    const uint32_t pl = fdiv(row, div_ir);
    const int h = (int)(row - pl * a.iR), me0 = h * a.iC + w0;
    const int ph_lo = h < k ? 0 : (int)fdiv((uint32_t)(h - k), div_s) + 1;
    // a row below the last window (floor-based output size: (iR - k) % s rows are covered by none)
    // has ph_lo == oR: both window rows are switched off and the reads clamped into the plane
    const bool row0 = ph_lo <= a.oR - 1, row1 = ph_lo + 1 <= a.oR - 1;
    const float *g = tog + pl * oplane;
    const int *x = tidx + pl * oplane;
    const int r0 = min(ph_lo, a.oR - 1) * a.oC, r1 = min(ph_lo + 1, a.oR - 1) * a.oC;
    int xi[2][NJ];
    float gv[2][NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      xi[0][j] = x[r0 + pc[j]]; gv[0][j] = g[r0 + pc[j]];
      xi[1][j] = x[r1 + pc[j]]; gv[1][j] = g[r1 + pc[j]];
    }
    pool_f4u acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const bool ok = cv[j] && (i == 0 ? row0 : row1);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // K3S2: an even element e sits in window columns e/2 and e/2 + 1 of the three, an odd one in (e+1)/2 only
          if (K3S2 && !((e & 1) ? j == (e + 1) / 2 : (j == e / 2 || j == e / 2 + 1))) continue;
          if (ok && xi[i][j] == me0 + e) acc[e] += gv[i][j];
        }
      }
    float *o = dst + (size_t)row * a.iC;
    if (relu_data) {
      const float *y = relu_data + (o - ig);
      if (nw == 4) {
        const pool_f4u yv = *reinterpret_cast<const pool_f4u *>(y);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = yv[e] > 0.0f ? acc[e] : 0.0f;
      } else {
        for (int e = 0; e < nw; ++e) acc[e] = y[e] > 0.0f ? acc[e] : 0.0f;
      }
    }
    if (nw == 4) {
      *reinterpret_cast<pool_f4u *>(o) = acc;
    } else {
      o[0] = acc[0];
      if (nw > 1) o[1] = acc[1];
      if (nw > 2) o[2] = acc[2];
    }
  }
}

// tuning knob pool_plane = 1 takes the plane-tiled kernels at any size (used by the tests on small shapes)
static bool force_pool_plane() { return tuning().pool_plane == 1; }

// planes per workgroup, within the LDS tile.  `backward`: plane_words = the staged (gradient, arg-max)
// pairs of a plane, work_words = the input-gradient elements it yields.
static int pool_planes_per_block(size_t plane_words, size_t work_words, size_t planes, bool backward) {
  // small tensors are launch-bound; the one-lane-per-element kernels finish them sooner
  if (planes * (plane_words > work_words ? plane_words : work_words) < (1u << 20) && !force_pool_plane()) return 0;
  if (plane_words == 0 || plane_words > (size_t)kPoolLdsWords) return 0;
  // at most 20 KB of LDS per workgroup where a plane allows it: eight workgroups share a compute
  // unit and their load and store phases overlap
  size_t pp = plane_words > 5120 ? 1 : 5120 / plane_words;
  // Measured on the CaffeNet layers (planes of 55 x 55, 27 x 27, 13 x 13): the forward kernel is
  // fastest with some 2300 staged inputs per workgroup (1 / 4 / 14 planes), the backward kernel
  // with some 8000 gradient elements but no more than sixteen planes (3 / 12 / 16).
  size_t want = backward ? (8192 + work_words - 1) / work_words : (2304 + plane_words - 1) / plane_words;
  if (want > 16) want = 16;
  if (pp > want) pp = want;
  if (pp > planes) pp = planes;
  return (int)(pp < 1 ? 1 : pp);
}

// ---- LRN (across channels) -----------------------------------------------------------------------
// scale^beta for the normalisation term scale = 1 + alpha/size * sum of squares.  The library
// routine powf costs more instructions than the rest of either kernel; two cheaper forms are used
// where they apply (chosen on the host, `mode` is uniform over a launch):
//   LRN_POW_34     beta == 0.75 (AlexNet / CaffeNet): sqrt(s) * sqrt(sqrt(s)), two correctly rounded
//                  square roots and one product;
//   LRN_POW_EXP2   any beta with alpha >= 0 (scale >= 1): exp2(beta * log2(s)) on the hardware
//                  transcendental units (1 ulp each; the exponent is small, so the error of the
//                  result stays within a few ulp);
//   LRN_POW_LIBM   everything else: powf.
// Reciprocals use v_rcp_f32 (1 ulp).  All of it is well inside the 1e-5 bar against the oracle's
// exact powf and double-precision reciprocals.
enum { LRN_POW_LIBM = 0, LRN_POW_34 = 1, LRN_POW_EXP2 = 2 };
__device__ __forceinline__ float lrn_pow(float s, float beta, int mode) {
  if (mode == LRN_POW_34) {
    const float r = __builtin_sqrtf(s);
    return r * __builtin_sqrtf(r);
  }
  if (mode == LRN_POW_EXP2) return __builtin_amdgcn_exp2f(beta * __builtin_amdgcn_logf(s));
  return powf(s, beta);
}
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
static int lrn_pow_mode(float alpha_over_size, float beta) {
  if (!(alpha_over_size >= 0.0f)) return LRN_POW_LIBM;  // scale could reach zero or below: keep powf's special cases
  if (beta == 0.75f) return LRN_POW_34;
  return LRN_POW_EXP2;
}

// forward: one lane per element sums the squares of its window [ch-w, ch+w] (clipped to the depth)
// in ascending channel order, then scale = 1 + alpha/size * sum and out = in / scale^beta; denoms
// keeps scale.  _f_lrn_forward carries a running window sum along the depth (src/kernels/lrn.hxx:
// 46-100); summing each window afresh differs from it by rounding only (a few ulp of the sum).
__global__ __launch_bounds__(TPB) void lrn_fwd_kernel(float *__restrict__ out, float *__restrict__ denoms,
                                                      const float *__restrict__ in, int rc, int D,
                                                      uint32_t total, int w, float aos, float beta,
                                                      int mode, FastDiv div_rc, FastDiv div_d) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  // e = (ib*D + ch)*rc + q
  const uint32_t t1 = fdiv(e, div_rc);
  const uint32_t ib = fdiv(t1, div_d);
  const int ch = t1 - ib * D;
  const int lo = max(0, ch - w), hi = min(D - 1, ch + w);
  const float *p = in + (size_t)e + (ptrdiff_t)(lo - ch) * rc;
  float sum = 0.0f, xv = 0.0f;
  for (int c = lo; c <= hi; ++c, p += rc) {
    const float x = *p;
    sum += x * x;
    if (c == ch) xv = x;
  }
  const float scale = aos * sum + 1.0f;
  denoms[e] = scale;
  out[e] = mode == LRN_POW_LIBM ? xv / powf(scale, beta) : xv * fast_rcp(lrn_pow(scale, beta, mode));
}

// backward as a gather over the window: in_grad[ch] = sum over od in [ch-w, ch+w] (ascending, the
// order in which _f_lrn_backward's od loop touches channel ch) of g(od,ch) * out_grad[od]
__global__ __launch_bounds__(TPB) void lrn_bwd_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                      const float *__restrict__ x, const float *__restrict__ den,
                                                      int rc, int D, uint32_t total, int w, float aos,
                                                      float beta, int mode, FastDiv div_rc, FastDiv div_d) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  // e = (ib*D + ch)*rc + q
  const uint32_t t1 = fdiv(e, div_rc);
  const uint32_t q = e - t1 * rc;
  const uint32_t ib = fdiv(t1, div_d);
  const int ch = t1 - ib * D;
  const size_t base = (size_t)ib * D * rc + q;
  const float xv = x[base + (size_t)ch * rc];
  float acc = 0.0f;
  for (int od = max(0, ch - w); od <= min(D - 1, ch + w); ++od) {
    const size_t o = base + (size_t)od * rc;
    const float dne = den[o];
    const float denom = lrn_pow(dne, beta, mode);
    float denom_n1, inv_denom;
    if (mode == LRN_POW_LIBM) {
      denom_n1 = (float)(1.0 / (double)(denom * dne));
      inv_denom = 0.0f;  // the centre term below takes the double-precision route
    } else {
      denom_n1 = fast_rcp(denom * dne);
      inv_denom = denom_n1 * dne;
    }
    const float wd = x[o];
    const float g2 = beta * denom_n1 * aos * 2 * wd;
    float gv;
    if (od == ch) gv = mode == LRN_POW_LIBM ? (float)(1.0 / (double)denom - (double)(g2 * xv)) : inv_denom - g2 * xv;
    else gv = -g2 * xv;
    acc += gv * og[o];
  }
  ig[e] = acc;
}

// Forward with one lane per (image, run of CH channels, four consecutive pixels of the plane): the
// CH + 2*WN inputs under the run are loaded once (all loads in flight together) and every channel's
// window is summed afresh from them in ascending channel order -- the sums lrn_fwd_kernel forms
// (terms outside the depth enter as +0, which leaves a sum of squares unchanged), a third of its
// loads and a fraction of its index arithmetic.  Every load and store moves 16 bytes (at dword
// alignment: planes of 27 x 27 or 13 x 13 floats start anywhere), so a wavefront touches 1 KB of a
// plane per instruction.  The last quad of a plane holds rc % 4 pixels and takes the scalar route.
typedef float lrn_f4u __attribute__((ext_vector_type(4), aligned(4)));
template <int WN, int CH, int MODE>
__global__ __launch_bounds__(TPB) void lrn_fwd_quad_kernel(float *__restrict__ out, float *__restrict__ denoms,
                                                           const float *__restrict__ in, int rc, int D,
                                                           uint32_t total, int nruns, int nqp, float aos,
                                                           float beta, FastDiv div_qp, FastDiv div_runs) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  // e = (ib*nruns + run)*nqp + quad
  const uint32_t t1 = fdiv(e, div_qp);
  const int q0 = 4 * (int)(e - t1 * nqp);
  const uint32_t ib = fdiv(t1, div_runs);
  const int c0 = (int)(t1 - ib * nruns) * CH;
  const size_t base = (size_t)ib * D * rc + q0;
  const int nv = min(4, rc - q0);  // pixels of this quad
  constexpr int NW = CH + 2 * WN;
  lrn_f4u xw[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int c = c0 - WN + i;
    const int cc = min(max(c, 0), D - 1);           // clamped: the load needs no branch
    const float *p = in + base + (size_t)cc * rc;
    lrn_f4u v;
    if (nv == 4) {
      v = *reinterpret_cast<const lrn_f4u *>(p);
    } else {
      v = lrn_f4u{p[0], nv > 1 ? p[1] : 0.0f, nv > 2 ? p[2] : 0.0f, 0.0f};
    }
    xw[i] = (c >= 0 && c < D) ? v : lrn_f4u{0.0f, 0.0f, 0.0f, 0.0f};
  }
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ch = c0 + c;
    if (ch >= D) break;
    lrn_f4u sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j <= 2 * WN; ++j) sum += xw[c + j] * xw[c + j];
    lrn_f4u scale, y;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      scale[t] = aos * sum[t] + 1.0f;
      y[t] = MODE == LRN_POW_LIBM ? xw[c + WN][t] / powf(scale[t], beta)
                                  : xw[c + WN][t] * fast_rcp(lrn_pow(scale[t], beta, MODE));
    }
    const size_t o = base + (size_t)ch * rc;
    if (nv == 4) {
      *reinterpret_cast<lrn_f4u *>(denoms + o) = scale;
      *reinterpret_cast<lrn_f4u *>(out + o) = y;
    } else {
#pragma unroll
      for (int t = 0; t < 3; ++t)
        if (t < nv) { denoms[o + t] = scale[t]; out[o + t] = y[t]; }
    }
  }
}

// The same gather with one lane per (image, pixel, run of CH channels): the per-channel terms of
// the window (scale^beta, the factor g2, x and out_grad) are computed once per lane and reused by
// the up to 2*WN+1 output channels that touch them, instead of once per (channel, window slot).
// Every product and sum is the one lrn_bwd_kernel forms, in the same order: identical results.
template <int WN, int CH, int MODE>
__global__ __launch_bounds__(TPB) void lrn_bwd_run_kernel(float *__restrict__ ig, const float *__restrict__ og,
                                                          const float *__restrict__ x,
                                                          const float *__restrict__ den, int rc, int D,
                                                          uint32_t total, int nruns, float aos, float beta,
                                                          FastDiv div_rc, FastDiv div_runs) {
  // neighbouring runs share their halo channels (three tensors' worth here): each XCD walks a
  // contiguous range of lanes so that the second reader of a halo finds it in its own L2 (measured:
  // 56 -> 51 us on the CaffeNet shapes; the forward kernel, with one input tensor, loses by it)
  const uint32_t e = xcd_remap(blockIdx.x, gridDim.x) * TPB + threadIdx.x;
  if (e >= total) return;
  // e = (ib*nruns + run)*rc + q
  const uint32_t t1 = fdiv(e, div_rc);
  const uint32_t q = e - t1 * rc;
  const uint32_t ib = fdiv(t1, div_runs);
  const int c0 = (int)(t1 - ib * nruns) * CH;
  const size_t base = (size_t)ib * D * rc + q;
  constexpr int NW = CH + 2 * WN;
  // denom holds scale^beta (LRN_POW_LIBM: the centre term divides in double precision, as the
  // reference's formula does) or its reciprocal (the fast modes)
  float denom[NW], g2[NW], xw[NW], ow[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int od = c0 - WN + i;
    denom[i] = 1.0f; g2[i] = 0.0f; xw[i] = 0.0f; ow[i] = 0.0f;
    if (od >= 0 && od < D) {
      const size_t o = base + (size_t)od * rc;
      const float dne = den[o];
      const float dn = lrn_pow(dne, beta, MODE);
      float denom_n1;
      if (MODE == LRN_POW_LIBM) {
        denom_n1 = (float)(1.0 / (double)(dn * dne));
        denom[i] = dn;
      } else {
        denom_n1 = fast_rcp(dn * dne);
        denom[i] = denom_n1 * dne;
      }
      const float wd = x[o];
      g2[i] = beta * denom_n1 * aos * 2 * wd;
      xw[i] = wd;
      ow[i] = og[o];
    }
  }
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ch = c0 + c;
    if (ch >= D) break;
    const float xv = xw[c + WN];
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j <= 2 * WN; ++j) {
      const int od = ch - WN + j;
      if (od < 0 || od >= D) continue;
      const int i = c + j;
      float gv;
      if (j == WN) gv = MODE == LRN_POW_LIBM ? (float)(1.0 / (double)denom[i] - (double)(g2[i] * xv)) : denom[i] - g2[i] * xv;
      else gv = -g2[i] * xv;
      acc += gv * ow[i];
    }
    ig[base + (size_t)ch * rc] = acc;
  }
}

// ---- dropout -------------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void dropout_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                      const unsigned int *__restrict__ mask, float scale,
                                                      unsigned int thr, size_t n) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride)
    out[i] = in[i] * (mask[i] > thr ? 1.0f : 0.0f) * scale;
}

// counter-based uint32 stream (splitmix64 finaliser over seed, call number and word index)
__global__ __launch_bounds__(TPB) void rand_uint_kernel(unsigned int *__restrict__ buf, size_t n,
                                                        uint64_t seed, uint64_t call) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) {
    uint64_t z = seed * 0x9E3779B97F4A7C15ull + call * 0xD1B54A32D192ED03ull + i + 0x632BE59BD9B4E019ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    buf[i] = (unsigned int)(z >> 16);
  }
}

// ---- softmax loss: one workgroup per image ----------------------------------------------------------
// Probabilities, the image's loss and, if asked, the input gradient (prob - onehot) * factor of the backward
// pass in the same launch; the batch sum of the losses follows in softmax_loss_sum_kernel.
__global__ __launch_bounds__(TPB) void softmax_fwd_kernel(float *__restrict__ prob, const float *__restrict__ in,
                                                          const float *__restrict__ labels,
                                                          float *__restrict__ loss_per_image, int len,
                                                          float *__restrict__ in_grad, double factor) {
  __shared__ float scratch[8];
  const int ib = blockIdx.x, tid = threadIdx.x;
  const float *x = in + (size_t)ib * len;
  float *y = prob + (size_t)ib * len;
  float mx = -FLT_MAX;
  for (int i = tid; i < len; i += TPB) mx = fmaxf(mx, x[i]);
  mx = block_reduce<true>(mx, scratch);
  float s = 0.0f;
  for (int i = tid; i < len; i += TPB) s += expf(x[i] - mx);
  s = block_reduce<false>(s, scratch);
  // a label outside [0, len) (NaN included) is never used as an index: the image's loss is NaN and the
  // gradient subtracts no 1
  const float lf = labels[ib];
  const bool valid = lf >= 0.0f && lf < (float)len;
  const int label = valid ? (int)lf : -1;
  for (int i = tid; i < len; i += TPB) {
    const float pv = expf(x[i] - mx) / s;
    y[i] = pv;
    if (in_grad) in_grad[(size_t)ib * len + i] = (float)((double)(i == label ? pv - 1.0f : pv) * factor);
    if (i == label) loss_per_image[ib] = -logf(fmaxf(pv, FLT_MIN));
  }
  if (!valid && tid == 0) loss_per_image[ib] = __int_as_float(0x7fc00000);
}
// batch sum in ascending image order (the order the reference accumulates its scalar loss): the
// workgroup fetches the per-image losses TPB at a time, coalesced, and lane 0 adds them up in order
__global__ __launch_bounds__(TPB) void softmax_loss_sum_kernel(float *__restrict__ loss_sum,
                                                               const float *__restrict__ per_image, int batch) {
  __shared__ float part[TPB];
  float s = 0.0f;
  for (int base = 0; base < batch; base += TPB) {
    const int i = base + (int)threadIdx.x;
    part[threadIdx.x] = i < batch ? per_image[i] : 0.0f;
    __syncthreads();
    if (threadIdx.x == 0) {
      const int n = min(TPB, batch - base);
      for (int j = 0; j < n; ++j) s += part[j];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) *loss_sum = s;
}
// The whole batch in ONE workgroup of sixteen wavefronts, for problems of a few thousand scores (LeNet: 64
// images x 10 classes), where the launches cost more than the arithmetic: wavefront w takes images w, w + 16, ...; a lane takes
// classes lane, lane + 64, ... of the scores staged in LDS; maximum and sum by shuffle trees; the per-image losses meet in LDS and
// lane 0 adds them in ascending image order, as softmax_loss_sum_kernel does.  Same values as the
// two-launch form for at most 64 classes (one class per lane: the sum of exponentials is the same shuffle
// tree over the same lanes), equal to rounding beyond.
constexpr int kSoftmaxSmallBatch = 1024, kSoftmaxSmallScores = 8192, kSoftmaxSmallThreads = 1024;
__global__ __launch_bounds__(kSoftmaxSmallThreads) void softmax_loss_small_kernel(
    float *__restrict__ prob, const float *__restrict__ in, const float *__restrict__ labels, int len, int batch,
    float *__restrict__ in_grad, double factor, float *__restrict__ loss_sum) {
  __shared__ float xs[kSoftmaxSmallScores];   // all scores, fetched once, coalesced: the per-image passes read LDS
  __shared__ float loss_of[kSoftmaxSmallBatch];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < batch * len; i += kSoftmaxSmallThreads) xs[i] = in[i];
  __syncthreads();
  for (int ib = wave; ib < batch; ib += kSoftmaxSmallThreads / 64) {
    const float *x = xs + ib * len;
    float *y = prob + (size_t)ib * len;
    float mx = -FLT_MAX;
    for (int i = lane; i < len; i += 64) mx = fmaxf(mx, x[i]);
    mx = wave_max_f(mx);
    mx = __shfl(mx, 0, 64);
    float s = 0.0f;
    for (int i = lane; i < len; i += 64) s += expf(x[i] - mx);
    s = wave_sum_f(s);
    s = __shfl(s, 0, 64);
    const float lf = labels[ib];
    const bool valid = lf >= 0.0f && lf < (float)len;
    const int label = valid ? (int)lf : -1;
    for (int i = lane; i < len; i += 64) {
      const float pv = expf(x[i] - mx) / s;
      y[i] = pv;
      if (in_grad) in_grad[(size_t)ib * len + i] = (float)((double)(i == label ? pv - 1.0f : pv) * factor);
      if (i == label) loss_of[ib] = -logf(fmaxf(pv, FLT_MIN));
    }
    if (!valid && lane == 0) loss_of[ib] = __int_as_float(0x7fc00000);
  }
  __syncthreads();
  if (tid == 0) {
    float total = 0.0f;
    for (int j = 0; j < batch; ++j) total += loss_of[j];
    *loss_sum = total;
  }
}
__global__ __launch_bounds__(TPB) void softmax_bwd_kernel(float *__restrict__ ig, const float *__restrict__ prob,
                                                          const float *__restrict__ labels, int len,
                                                          uint32_t total, double factor, FastDiv div_len) {
  const uint32_t e = blockIdx.x * TPB + threadIdx.x;
  if (e >= total) return;
  const uint32_t ib = fdiv(e, div_len);
  const int i = e - ib * len;
  float v = prob[e];
  const float lf = labels[ib];
  if (lf >= 0.0f && lf < (float)len && i == (int)lf) v -= 1.0f;
  ig[e] = (float)((double)v * factor);
}

// ---- BLAS-1 / SGD ----------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void saxpby_kernel(size_t n, float a, const float *__restrict__ x, float b,
                                                     float *__restrict__ y, int has_b) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride)
    y[i] = has_b ? a * x[i] + b * y[i] : a * x[i] + y[i];
}
__global__ __launch_bounds__(TPB) void l1_update_kernel(int n, float *__restrict__ g, float lambda,
                                                        const float *__restrict__ w) {
  const int i = blockIdx.x * TPB + threadIdx.x;
  if (i < n) g[i] += lambda * (w[i] > 0 ? 1.0f : -1.0f);
}
// one pass: the three BLAS-1 calls of SGDGradientUpdater::update applied per element in the same
// order, each product/sum rounded to fp32 as the separate calls would
__device__ __forceinline__ void sgd_element(float *__restrict__ w, float *__restrict__ g, float *__restrict__ h,
                                            size_t i, float step, float mom, float lambda, int l1) {
  const float wi = w[i];
  float gi = g[i];
  if (lambda != 0.0f) {
    gi = l1 ? gi + lambda * (wi > 0 ? 1.0f : -1.0f) : __fadd_rn(__fmul_rn(lambda, wi), gi);
    g[i] = gi;
  }
  const float hi = __fadd_rn(__fmul_rn(step, gi), __fmul_rn(mom, h[i]));
  h[i] = hi;
  w[i] = __fadd_rn(__fmul_rn(-1.0f, hi), wi);
}
__global__ __launch_bounds__(TPB) void sgd_kernel(size_t n, float *__restrict__ w, float *__restrict__ g,
                                                  float *__restrict__ h, float step, float mom, float lambda,
                                                  int l1) {
  const size_t stride = (size_t)gridDim.x * TPB;
  for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride)
    sgd_element(w, g, h, i, step, mom, lambda, l1);
}

// Several small tensors in one launch (the biases and small filters of a network: a launch each
// costs more than their update).  The job table travels as a kernel argument; a workgroup handles
// kSgdChunk elements of one job, found from the first-block table.
constexpr int kSgdBatch = 16, kSgdChunk = TPB * 2;  // (two elements per lane: LeNet's one launch 8.6 -> 5 us against eight)
struct SgdBatch {
  cct_sgd_job job[kSgdBatch];
  uint32_t first_block[kSgdBatch + 1];
  int count;
};
__global__ __launch_bounds__(TPB) void sgd_batch_kernel(const SgdBatch b) {
  int j = 0;
  while (j + 1 < b.count && blockIdx.x >= b.first_block[j + 1]) ++j;
  const cct_sgd_job &job = b.job[j];
  const size_t i0 = (size_t)(blockIdx.x - b.first_block[j]) * kSgdChunk;
  const size_t i1 = i0 + kSgdChunk < job.n ? i0 + kSgdChunk : job.n;
  for (size_t i = i0 + threadIdx.x; i < i1; i += TPB)
    sgd_element(job.model, job.gradient, job.history, i, job.stepsize, job.momentum, job.lambda, job.l1);
}

// ---- gemv (row-major M x N, lda = N) -------------------------------------------------------------------
// NoTrans: one workgroup per output row; Trans: one lane per output column
__global__ __launch_bounds__(TPB) void gemv_n_kernel(int M, int N, float alpha, const float *__restrict__ A,
                                                     const float *__restrict__ x, float beta,
                                                     float *__restrict__ y) {
  __shared__ float scratch[8];
  const int row = blockIdx.x;
  float s = 0.0f;
  for (int j = threadIdx.x; j < N; j += TPB) s += A[(size_t)row * N + j] * x[j];
  s = block_reduce<false>(s, scratch);
  if (threadIdx.x == 0) y[row] = (beta == 0.0f) ? alpha * s : alpha * s + beta * y[row];
}
__global__ __launch_bounds__(TPB) void gemv_t_kernel(int M, int N, float alpha, const float *__restrict__ A,
                                                     const float *__restrict__ x, float beta,
                                                     float *__restrict__ y) {
  const int col = blockIdx.x * TPB + threadIdx.x;
  if (col >= N) return;
  float s = 0.0f;
  for (int i = 0; i < M; ++i) s += A[(size_t)i * N + col] * x[i];
  y[col] = (beta == 0.0f) ? alpha * s : alpha * s + beta * y[col];
}

static inline uint32_t grid_stride_blocks(size_t n) {
  const size_t want = (n + TPB - 1) / TPB;
  const size_t cap = 256 * 32;  // 32 workgroups per compute unit
  return (uint32_t)(want < cap ? (want ? want : 1) : cap);
}

}  // namespace cct

using namespace cct;

extern "C" {

int cct_hip_memset(void *dev_ptr, int value, size_t size_in_byte) {
  CCT_ENSURE_INIT();
  if (size_in_byte == 0) return 0;
  CCT_REQUIRE(dev_ptr, "memset: null pointer");
  const unsigned char b = (unsigned char)value;
  if ((uintptr_t)dev_ptr % 4 == 0 && size_in_byte % 4 == 0) {
    const uint32_t w = b * 0x01010101u;
    float f;
    memcpy(&f, &w, 4);
    const size_t n = size_in_byte / 4;
    hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream,
                       (float *)dev_ptr, n, f);
  } else {
    hipLaunchKernelGGL(fill_u8_kernel, dim3(grid_stride_blocks(size_in_byte)), dim3(TPB), 0, ctx().stream,
                       (unsigned char *)dev_ptr, size_in_byte, b);
  }
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_sconstant_initialize(float *arr, size_t n, float value) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(arr, "sconstant_initialize: null pointer");
  hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, arr, n, value);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_remap(float *dst, const float *src, const cct_pmap_helper *a) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dst && src && a, "remap: null argument");
  const size_t rc = a->sR * a->sC, slices = a->sD * a->sB;
  if (rc == 0 || slices == 0) return 0;
  CCT_REQUIRE(slices < (1ull << 31) && rc < (1ull << 31), "remap: too many slices");
  const char *d0 = (const char *)dst, *s0 = (const char *)src;
  const size_t bytes = rc * slices * 4;
  CCT_REQUIRE(d0 + bytes <= s0 || s0 + bytes <= d0, "remap: dst and src overlap");
  // parts per slice: each lane moves up to 64 bytes; few slices with long rows are cut further
  uint32_t gy = (uint32_t)((rc / 4 + 4 * TPB - 1) / (4 * TPB));
  if (gy < 1) gy = 1;
  if (gy > 64) gy = 64;
  hipLaunchKernelGGL(remap_kernel, dim3((uint32_t)slices, gy), dim3(TPB), 0, ctx().stream, dst, src,
                     (uint32_t)rc, (uint32_t)a->sD, make_fastdiv((uint32_t)a->sB));
  CCT_LAUNCH_CHECK();
  note_kernel("remap_kernel");
  return 0;
}

int cct_hip_remap_bias_backward(float *dst, const float *src, const cct_pmap_helper *a, float *bias_grad) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dst && src && a && bias_grad, "remap_bias_backward: null argument");
  const size_t rc = a->sR * a->sC, slices = a->sD * a->sB;
  if (a->sB == 0) return 0;
  if (rc == 0 || a->sD == 0) return cct_hip_sconstant_initialize(bias_grad, a->sB, 0.0f);
  CCT_REQUIRE(slices < (1ull << 31) && rc < (1ull << 31), "remap_bias_backward: too many slices");
  const char *d0 = (const char *)dst, *s0 = (const char *)src;
  const size_t bytes = rc * slices * 4;
  CCT_REQUIRE(d0 + bytes <= s0 || s0 + bytes <= d0, "remap_bias_backward: dst and src overlap");
  uint32_t gy = (uint32_t)((rc / 4 + 4 * TPB - 1) / (4 * TPB));
  if (gy < 1) gy = 1;
  if (gy > 64) gy = 64;
  void *ws = nullptr;
  int rc_ws = get_workspace(slices * gy * sizeof(float), &ws);
  if (rc_ws) return rc_ws;
  hipLaunchKernelGGL(remap_bias_kernel, dim3((uint32_t)slices, gy), dim3(TPB), 0, ctx().stream, dst, src,
                     (uint32_t)rc, (uint32_t)a->sD, make_fastdiv((uint32_t)a->sB), (float *)ws);
  CCT_LAUNCH_CHECK();
  hipLaunchKernelGGL(bias_partial_sum_kernel, dim3((uint32_t)a->sB), dim3(TPB), 0, ctx().stream, bias_grad,
                     (const float *)ws, (uint32_t)a->sB, (uint32_t)a->sD, gy);
  CCT_LAUNCH_CHECK();
  note_kernel("remap_bias_kernel");
  return 0;
}

int cct_hip_copy_depth_slice(float *part, float *whole, int B, int d_total, int d_off, int d_count, size_t rc,
                             int gather) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(part && whole, "copy_depth_slice: null argument");
  CCT_REQUIRE(B >= 0 && d_total > 0 && d_off >= 0 && d_count > 0 && d_off + d_count <= d_total && rc > 0,
              "copy_depth_slice: bad slice [%d, %d) of %d", d_off, d_off + d_count, d_total);
  CCT_REQUIRE((size_t)d_total * rc < (1ull << 31) && B <= 65535, "copy_depth_slice: tensor too large");
  if (B == 0) return 0;
  const uint32_t per_image = (uint32_t)(d_count * rc);
  uint32_t gx = (per_image + TPB - 1) / TPB;
  if (gx > 1024) gx = 1024;
  hipLaunchKernelGGL(depth_slice_kernel, dim3(gx, B), dim3(TPB), 0, ctx().stream, part, whole, per_image,
                     (uint32_t)(d_total * rc), (uint32_t)(d_off * rc), gather);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_forward_bias(const float *bias, float *out, int fmap_size, int depth, int batch_size) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(bias && out, "forward_bias: null argument");
  CCT_REQUIRE(fmap_size > 0 && depth > 0 && batch_size >= 0, "forward_bias: bad sizes");
  if (batch_size == 0) return 0;
  const size_t slices = (size_t)depth * batch_size;
  CCT_REQUIRE(slices < (1ull << 31), "forward_bias: too many slices");
  if (fmap_size < 128 && slices * (size_t)fmap_size < (1ull << 31)) {
    const uint32_t total = (uint32_t)(slices * fmap_size);
    hipLaunchKernelGGL(bias_forward_flat_kernel, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, out, bias,
                       total, make_fastdiv((uint32_t)fmap_size), make_fastdiv((uint32_t)depth));
    CCT_LAUNCH_CHECK();
    return 0;
  }
  uint32_t gy = (uint32_t)((fmap_size + TPB - 1) / TPB);
  if (gy > 64) gy = 64;
  hipLaunchKernelGGL(bias_forward_kernel, dim3((uint32_t)slices, gy), dim3(TPB), 0, ctx().stream, out, bias,
                     (uint32_t)fmap_size, make_fastdiv((uint32_t)depth));
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_backward_bias_fc(float *bias_grad, const float *out_grad, int D, int B) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(bias_grad && out_grad && D > 0 && B >= 0, "backward_bias_fc: bad argument");
  static_assert(TPB == 256, "bias_backward_fc_kernel: four wavefronts per workgroup");
  hipLaunchKernelGGL(bias_backward_fc_kernel, dim3((uint32_t)((D + 63) / 64)), dim3(TPB), 0, ctx().stream, bias_grad,
                     out_grad, D, B);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_relu_forward(float *out, const float *in, size_t n) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(out && in, "relu_forward: null argument");
  hipLaunchKernelGGL(relu_fwd_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, out, in, n);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_relu_backward(float *in_grad, const float *out_grad, const float *in_data, size_t n) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(in_grad && out_grad && in_data, "relu_backward: null argument");
  hipLaunchKernelGGL(relu_bwd_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, in_grad,
                     out_grad, in_data, n);
  CCT_LAUNCH_CHECK();
  return 0;
}

static int check_pool(const cct_pool_args *a, const char *who) {
  CCT_REQUIRE(a && a->max_index, "%s: null argument", who);
  CCT_REQUIRE(a->stride >= 1 && a->kernel_size >= 1 && a->iR >= 1 && a->iC >= 1 && a->oR >= 1 && a->oC >= 1 &&
                  a->D >= 0 && a->B >= 0,
              "%s: bad sizes", who);
  // every window must start inside the input, as the reference's floor-based output size guarantees
  CCT_REQUIRE((a->oR - 1) * a->stride < a->iR && (a->oC - 1) * a->stride < a->iC,
              "%s: output %dx%d does not fit input %dx%d", who, a->oR, a->oC, a->iR, a->iC);
  CCT_REQUIRE((size_t)a->D * a->B * a->iR * a->iC < (1ull << 31), "%s: tensor too large", who);
  return 0;
}

int cct_hip_maxpool_forward(float *out, const float *in, const cct_pool_args *a) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out && in, "maxpool_forward: null argument");
  int rc = check_pool(a, "maxpool_forward");
  if (rc) return rc;
  const size_t total = (size_t)a->D * a->B * a->oR * a->oC;
  if (total == 0) return 0;
  const size_t planes = (size_t)a->D * a->B, iplane = (size_t)a->iR * a->iC, oplane = (size_t)a->oR * a->oC;
  if (const int pp = pool_planes_per_block(iplane, oplane, planes, false)) {
    hipLaunchKernelGGL(maxpool_fwd_plane_kernel, dim3((uint32_t)((planes + pp - 1) / pp)), dim3(TPB),
                       (size_t)pp * iplane * sizeof(float), ctx().stream,
                       out, a->max_index, in, *a, (uint32_t)planes, pp, make_fastdiv(a->oC),
                       make_fastdiv((uint32_t)oplane));
    CCT_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(maxpool_fwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, out,
                     a->max_index, in, *a, (uint32_t)total, make_fastdiv(a->oC), make_fastdiv(a->oR));
  CCT_LAUNCH_CHECK();
  return 0;
}

// relu_data: mask the result with (relu_data > 0) (same shape as in_grad); pooled: mask every
// window's gradient with (pooled > 0) (same shape as out_grad) -- at most one of the two
static int maxpool_backward_impl(float *in_grad, const float *out_grad, const cct_pool_args *a,
                                 const float *relu_data, const float *pooled = nullptr) {
  CCT_REQUIRE(in_grad && out_grad, "maxpool_backward: null argument");
  int rc = check_pool(a, "maxpool_backward");
  if (rc) return rc;
  const size_t total = (size_t)a->D * a->B * a->iR * a->iC;
  if (total == 0) return 0;
  const size_t planes = (size_t)a->D * a->B, iplane = (size_t)a->iR * a->iC, oplane = (size_t)a->oR * a->oC;
  const int pp = pool_planes_per_block(2 * oplane, iplane, planes, true);
  const bool quad = pp && a->stride >= 2 && a->kernel_size <= 2 * a->stride && a->iC <= 256;
  if (pooled && !quad) {
    // the other kernels do not switch windows off while they stage: a pass over the (small) output
    // gradient does it first, into the library's workspace
    void *ws = nullptr;
    rc = get_workspace(planes * oplane * sizeof(float), &ws);
    if (rc) return rc;
    hipLaunchKernelGGL(mask_positive_kernel, dim3(grid_stride_blocks(planes * oplane)), dim3(TPB), 0, ctx().stream,
                       (float *)ws, out_grad, pooled, planes * oplane);
    CCT_LAUNCH_CHECK();
    out_grad = (const float *)ws;
    pooled = nullptr;
  }
  if (pp) {
    const dim3 grid((uint32_t)((planes + pp - 1) / pp));
    if (quad) {
      int lpr_shift = 0;
      while ((4 << lpr_shift) < a->iC) ++lpr_shift;
      if (a->kernel_size == 3 && a->stride == 2)
        hipLaunchKernelGGL(maxpool_bwd_quad_kernel<true>, grid, dim3(TPB), (size_t)2 * pp * oplane * sizeof(float),
                           ctx().stream, in_grad, out_grad, a->max_index, *a, (uint32_t)planes, pp, lpr_shift,
                           make_fastdiv(a->iR), make_fastdiv(a->stride), relu_data, pooled);
      else
        hipLaunchKernelGGL(maxpool_bwd_quad_kernel<false>, grid, dim3(TPB), (size_t)2 * pp * oplane * sizeof(float),
                           ctx().stream, in_grad, out_grad, a->max_index, *a, (uint32_t)planes, pp, lpr_shift,
                           make_fastdiv(a->iR), make_fastdiv(a->stride), relu_data, pooled);
      relu_data = nullptr;  // done inside the kernel
    } else if (a->kernel_size <= 2 * a->stride)
      hipLaunchKernelGGL(maxpool_bwd_plane_kernel<true>, grid, dim3(TPB), 0, ctx().stream, in_grad, out_grad,
                         a->max_index, *a, (uint32_t)planes, pp, make_fastdiv(a->iC), make_fastdiv((uint32_t)iplane),
                         make_fastdiv(a->stride));
    else
      hipLaunchKernelGGL(maxpool_bwd_plane_kernel<false>, grid, dim3(TPB), 0, ctx().stream, in_grad, out_grad,
                         a->max_index, *a, (uint32_t)planes, pp, make_fastdiv(a->iC), make_fastdiv((uint32_t)iplane),
                         make_fastdiv(a->stride));
    CCT_LAUNCH_CHECK();
    // the other kernels do not mask: a separate pass does
    return relu_data ? cct_hip_relu_backward(in_grad, in_grad, relu_data, total) : 0;
  }
  if (a->kernel_size <= 2 * a->stride)
    hipLaunchKernelGGL(maxpool_bwd_kernel<true>, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, in_grad,
                       out_grad, a->max_index, *a, (uint32_t)total, make_fastdiv(a->iC), make_fastdiv(a->iR));
  else
    hipLaunchKernelGGL(maxpool_bwd_kernel<false>, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, in_grad,
                       out_grad, a->max_index, *a, (uint32_t)total, make_fastdiv(a->iC), make_fastdiv(a->iR));
  CCT_LAUNCH_CHECK();
  return relu_data ? cct_hip_relu_backward(in_grad, in_grad, relu_data, total) : 0;
}

int cct_hip_maxpool_backward(float *in_grad, const float *out_grad, const cct_pool_args *a) {
  CCT_ENSURE_INIT();
  return maxpool_backward_impl(in_grad, out_grad, a, nullptr);
}

int cct_hip_maxpool_backward_relu(float *in_grad, const float *out_grad, const cct_pool_args *a,
                                  const float *relu_data) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(relu_data, "maxpool_backward_relu: null activation tensor");
  return maxpool_backward_impl(in_grad, out_grad, a, relu_data);
}

int cct_hip_maxpool_backward_relu_pooled(float *in_grad, const float *out_grad, const cct_pool_args *a,
                                         const float *pooled) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(pooled, "maxpool_backward_relu_pooled: null pooled tensor");
  return maxpool_backward_impl(in_grad, out_grad, a, nullptr, pooled);
}

int cct_hip_lrn_forward(float *out, const float *in, const cct_lrn_forward_args *a,
                        const cct_lrn_forward_normalize_args *a2) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out && in && a && a2 && a->denoms, "lrn_forward: null argument");
  CCT_REQUIRE(a->iR > 0 && a->iC > 0 && a->iD > 0 && a->iB >= 0 && a->norm_window >= 0, "lrn_forward: bad sizes");
  const size_t total = (size_t)a->iB * a->iD * a->iR * a->iC;
  CCT_REQUIRE(total < (1ull << 31), "lrn_forward: tensor too large");
  if (total == 0) return 0;
  const int mode = lrn_pow_mode(a2->alpha_over_size, a2->beta);
  if (a->norm_window == 2) {
    // Four pixels per lane and a run of CH channels: the longest run (fewest halo loads: CH + 4 loads
    // per CH outputs) that still leaves some six workgroups per compute unit; the kernel runs for
    // 25-50 us and is latency-bound below that (CaffeNet: norm1 runs of 8, norm2 runs of 4).
    const int rc = a->iR * a->iC, nqp = (rc + 3) / 4;
    const size_t want = (size_t)6 * TPB * (ctx().compute_units > 0 ? ctx().compute_units : 256);
    int ch = 16;
    while (ch > 4 && (size_t)a->iB * ((a->iD + ch - 1) / ch) * nqp < want) ch >>= 1;
    const int nruns = (a->iD + ch - 1) / ch;
    const size_t lanes = (size_t)a->iB * nruns * nqp;
#define CCT_LRN_FWD_CH(MODE, CH)                                                                                \
  hipLaunchKernelGGL((lrn_fwd_quad_kernel<2, CH, MODE>), dim3(blocks_for(lanes)), dim3(TPB), 0, ctx().stream, out, \
                     (float *)a->denoms, in, rc, a->iD, (uint32_t)lanes, nruns, nqp, a2->alpha_over_size, a2->beta, \
                     make_fastdiv(nqp), make_fastdiv(nruns))
#define CCT_LRN_FWD(MODE)                      \
  do {                                         \
    if (ch == 16) CCT_LRN_FWD_CH(MODE, 16);    \
    else if (ch == 8) CCT_LRN_FWD_CH(MODE, 8); \
    else CCT_LRN_FWD_CH(MODE, 4);              \
  } while (0)
    if (mode == LRN_POW_34) CCT_LRN_FWD(LRN_POW_34);
    else if (mode == LRN_POW_EXP2) CCT_LRN_FWD(LRN_POW_EXP2);
    else CCT_LRN_FWD(LRN_POW_LIBM);
#undef CCT_LRN_FWD_CH
#undef CCT_LRN_FWD
    CCT_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(lrn_fwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, out,
                     (float *)a->denoms, in, a->iR * a->iC, a->iD, (uint32_t)total, a->norm_window,
                     a2->alpha_over_size, a2->beta, mode, make_fastdiv(a->iR * a->iC), make_fastdiv(a->iD));
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_lrn_backward(float *in_grad, const float *out_grad, const cct_lrn_backward_args *a) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(in_grad && out_grad && a && a->denoms && a->input_data, "lrn_backward: null argument");
  CCT_REQUIRE(a->oR > 0 && a->oC > 0 && a->oD > 0 && a->oB >= 0 && a->norm_window >= 0, "lrn_backward: bad sizes");
  const size_t total = (size_t)a->oB * a->oD * a->oR * a->oC;
  CCT_REQUIRE(total < (1ull << 31), "lrn_backward: tensor too large");
  if (total == 0) return 0;
  const int mode = lrn_pow_mode(a->alpha_over_size, a->beta);
  if (a->norm_window == 2) {
    // one pixel per lane, runs of eight channels: with four tensors' worth of registers per window
    // slot, two or four pixels per lane measured 10-40 % slower
    constexpr int CH = 8;
    const int nruns = (a->oD + CH - 1) / CH;
    const size_t lanes = (size_t)a->oB * nruns * a->oR * a->oC;
#define CCT_LRN_BWD(MODE)                                                                                       \
  hipLaunchKernelGGL((lrn_bwd_run_kernel<2, CH, MODE>), dim3(blocks_for(lanes)), dim3(TPB), 0, ctx().stream,    \
                     in_grad, out_grad, (const float *)a->input_data, (const float *)a->denoms, a->oR * a->oC,  \
                     a->oD, (uint32_t)lanes, nruns, a->alpha_over_size, a->beta, make_fastdiv(a->oR * a->oC),   \
                     make_fastdiv(nruns))
    if (mode == LRN_POW_34) CCT_LRN_BWD(LRN_POW_34);
    else if (mode == LRN_POW_EXP2) CCT_LRN_BWD(LRN_POW_EXP2);
    else CCT_LRN_BWD(LRN_POW_LIBM);
#undef CCT_LRN_BWD
    CCT_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(lrn_bwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, in_grad, out_grad,
                     (const float *)a->input_data, (const float *)a->denoms, a->oR * a->oC, a->oD,
                     (uint32_t)total, a->norm_window, a->alpha_over_size, a->beta, mode,
                     make_fastdiv(a->oR * a->oC), make_fastdiv(a->oD));
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_dropout_forward_train(float *out, const float *in, const unsigned int *mask, float scale,
                                  unsigned int threshold, size_t n) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(out && in && mask, "dropout_forward_train: null argument");
  hipLaunchKernelGGL(dropout_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, out, in, mask,
                     scale, threshold, n);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_init_rng(int random_seed) {
  CCT_ENSURE_INIT();
  ctx().rng_seed = (uint64_t)(int64_t)random_seed;
  ctx().rng_calls = 0;
  return 0;
}

int cct_hip_rand_uint_initialize(unsigned int *buf, int n) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(n >= 0, "rand_uint_initialize: negative count");
  if (n == 0) return 0;
  CCT_REQUIRE(buf, "rand_uint_initialize: null buffer");
  hipLaunchKernelGGL(rand_uint_kernel, dim3(grid_stride_blocks((size_t)n)), dim3(TPB), 0, ctx().stream, buf,
                     (size_t)n, ctx().rng_seed, ctx().rng_calls);
  CCT_LAUNCH_CHECK();
  ctx().rng_calls++;
  return 0;
}

static int softmax_loss_launch(float *prob, const float *in, const float *labels, float *loss_sum, float *in_grad,
                               int len_per_image, int batch, int spatial, const char *what) {
  CCT_REQUIRE(prob && in && labels && loss_sum, "%s: null argument", what);
  CCT_REQUIRE(len_per_image > 0 && batch >= 0 && spatial > 0, "%s: bad sizes", what);
  CCT_REQUIRE((size_t)len_per_image * (size_t)(batch > 0 ? batch : 1) < (1ull << 31), "%s: tensor too large", what);
  const double factor = 1. / (double)(batch > 0 ? batch : 1) / (double)spatial;
  if (batch > 0 && batch <= kSoftmaxSmallBatch && (size_t)batch * len_per_image <= (size_t)kSoftmaxSmallScores) {
    hipLaunchKernelGGL(softmax_loss_small_kernel, dim3(1), dim3(kSoftmaxSmallThreads), 0, ctx().stream, prob, in, labels, len_per_image,
                       batch, in_grad, factor, loss_sum);
    CCT_LAUNCH_CHECK();
    return 0;
  }
  void *ws = nullptr;
  int rc = get_workspace((size_t)(batch > 0 ? batch : 1) * sizeof(float), &ws);
  if (rc) return rc;
  if (batch > 0) {
    hipLaunchKernelGGL(softmax_fwd_kernel, dim3(batch), dim3(TPB), 0, ctx().stream, prob, in, labels, (float *)ws,
                       len_per_image, in_grad, factor);
    CCT_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(softmax_loss_sum_kernel, dim3(1), dim3(TPB), 0, ctx().stream, loss_sum, (const float *)ws, batch);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_softmax_loss_forward(float *prob, const float *in, const float *labels, float *loss_sum,
                                 int len_per_image, int batch) {
  CCT_ENSURE_INIT();
  return softmax_loss_launch(prob, in, labels, loss_sum, nullptr, len_per_image, batch, 1, "softmax_loss_forward");
}

int cct_hip_softmax_loss_forward_backward(float *prob, float *in_grad, const float *in, const float *labels,
                                          float *loss_sum, int len_per_image, int batch, int spatial) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(in_grad, "softmax_loss_forward_backward: null gradient");
  return softmax_loss_launch(prob, in, labels, loss_sum, in_grad, len_per_image, batch, spatial,
                             "softmax_loss_forward_backward");
}

int cct_hip_softmax_loss_backward(float *in_grad, const float *prob, const float *labels, int len_per_image,
                                  int batch, int spatial) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(in_grad && prob && labels, "softmax_loss_backward: null argument");
  CCT_REQUIRE(len_per_image > 0 && batch > 0 && spatial > 0, "softmax_loss_backward: bad sizes");
  const size_t total = (size_t)len_per_image * batch;
  CCT_REQUIRE(total < (1ull << 31), "softmax_loss_backward: tensor too large");
  const double factor = 1. / (double)batch / (double)spatial;
  hipLaunchKernelGGL(softmax_bwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, ctx().stream, in_grad, prob,
                     labels, len_per_image, (uint32_t)total, factor, make_fastdiv(len_per_image));
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_math_saxpby(size_t n, float alpha, const float *x, float beta, float *y) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(x && y, "math_saxpby: null argument");
  hipLaunchKernelGGL(saxpby_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, n, alpha, x, beta,
                     y, 1);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_math_saxpy(size_t n, float alpha, const float *x, float *y) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(x && y, "math_saxpy: null argument");
  hipLaunchKernelGGL(saxpby_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, n, alpha, x, 1.0f,
                     y, 0);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_L1_update(int n, float *gradient, float lambda, const float *model) {
  CCT_ENSURE_INIT();
  if (n <= 0) return 0;
  CCT_REQUIRE(gradient && model, "L1_update: null argument");
  hipLaunchKernelGGL(l1_update_kernel, dim3(blocks_for(n)), dim3(TPB), 0, ctx().stream, n, gradient, lambda,
                     model);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_sgd_update(size_t n, float *model, float *gradient, float *history, float stepsize, float momentum,
                       float lambda, int l1) {
  CCT_ENSURE_INIT();
  if (n == 0) return 0;
  CCT_REQUIRE(model && gradient && history, "sgd_update: null argument");
  hipLaunchKernelGGL(sgd_kernel, dim3(grid_stride_blocks(n)), dim3(TPB), 0, ctx().stream, n, model, gradient,
                     history, stepsize, momentum, lambda, l1);
  CCT_LAUNCH_CHECK();
  return 0;
}

int cct_hip_sgd_update_batch(const cct_sgd_job *jobs, int count) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(count >= 0 && (jobs || count == 0), "sgd_update_batch: null job table");
  for (int at = 0; at < count;) {
    SgdBatch b;
    b.count = 0;
    uint32_t blocks = 0;
    for (; at < count && b.count < kSgdBatch; ++at) {
      const cct_sgd_job &j = jobs[at];
      if (j.n == 0) continue;
      CCT_REQUIRE(j.model && j.gradient && j.history, "sgd_update_batch: null argument in job %d", at);
      CCT_REQUIRE(j.n < ((size_t)1 << 40), "sgd_update_batch: job %d too large", at);
      b.job[b.count] = j;
      b.first_block[b.count] = blocks;
      blocks += (uint32_t)((j.n + kSgdChunk - 1) / kSgdChunk);
      ++b.count;
    }
    if (b.count == 0) continue;
    b.first_block[b.count] = blocks;
    hipLaunchKernelGGL(sgd_batch_kernel, dim3(blocks), dim3(TPB), 0, ctx().stream, b);
    CCT_LAUNCH_CHECK();
  }
  return 0;
}

int cct_hip_sgemv(int TA, int M, int N, float alpha, const float *A, const float *x, float beta, float *y) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(TA == CCT_NO_TRANS || TA == CCT_TRANS, "sgemv: bad transpose flag %d", TA);
  CCT_REQUIRE(M >= 0 && N >= 0, "sgemv: negative dimension");
  if (M == 0 || N == 0) return 0;
  CCT_REQUIRE(A && x && y, "sgemv: null argument");
  if (TA == CCT_NO_TRANS)
    hipLaunchKernelGGL(gemv_n_kernel, dim3(M), dim3(TPB), 0, ctx().stream, M, N, alpha, A, x, beta, y);
  else
    hipLaunchKernelGGL(gemv_t_kernel, dim3(blocks_for(N)), dim3(TPB), 0, ctx().stream, M, N, alpha, A, x, beta,
                       y);
  CCT_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
