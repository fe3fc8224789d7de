// Convolutions with a very short contraction and few output maps (LeNet's first layer: one 28 x 28 channel,
// twenty 5 x 5 filters, batch 64): forward and weight / bias gradient as plain fp32 multiply-adds.
//
// These are the GEMMs of ConvolutionBridge::forward_dev / backward_dev
// (src/bridges/ConvolutionBridge_impl.hxx:294-373, 551-628) for a layer whose lowered matrix has k*k*d = 25 rows
// and whose model has 20: a 32-row MFMA tile with a K loop of 25 is mostly padding, prologue and epilogue, and the
// weight gradient needs a partial-sum pass on top.  Here
//   forward : one lane per output pixel; its d*k*k source values sit in registers, the filters are staged in LDS
//             once per workgroup (every lane of a wavefront needs the same weights at the same time: 16-byte
//             broadcast reads), one store per map;
//   weights : one workgroup per (map, group of images); a lane takes a pixel or two of the group with d*k*k
//             accumulators (+ 1 for the bias gradient), the workgroup adds them up in a fixed order (lane tree, then
//             the wavefronts in order) and a second launch adds the groups in order -- no atomics, run-to-run
//             identical.
// The data gradient of such a layer (not needed for a first layer) stays with the other kernels.
//
// Bound: launch latency (the arithmetic is 37 MFLOP per product for LeNet conv1 at batch 64); algorithmic bytes are the
// input, the output (or its gradient) and the filters, each once.
#include "cct_common.h"
#include "mfma_common.h"

namespace cct {

constexpr int kConvSmallMaxMaps = 32;
constexpr int CS_THREADS = 256;

// Sum over the 64 lanes of a wavefront, valid in lane 63, as data-parallel-primitive moves (no LDS traffic):
// neighbours within quads, quads within rows of 16 (half-row and row mirrors), then row 0 -> 1, 2 -> 3 and
// rows 0..1 -> 2..3 through the rows' last lanes.  A fixed order: run-to-run identical.
__device__ __forceinline__ float conv_small_wave_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));
  return v;
}

// LDS row of one map's filters: d*k*k floats padded to whole 16-byte reads
template <int KS, int D>
struct ConvSmallShape {
  static constexpr int KK = KS * KS, DKK = D * KK, ROW = (DKK + 3) / 4 * 4;
};

template <int KS, int D>
__global__ __launch_bounds__(CS_THREADS) void conv_small_forward_kernel(float *__restrict__ out,
                                                                       const float *__restrict__ in,
                                                                       const float *__restrict__ w,
                                                                       const float *__restrict__ bias, int n, int pad,
                                                                       int o, int m, uint32_t total, FastDiv div_mm,
                                                                       FastDiv div_m, int relu) {
  constexpr int DKK = ConvSmallShape<KS, D>::DKK, ROW = ConvSmallShape<KS, D>::ROW;
  // the filters (and the bias behind each), in LDS: every lane of a wavefront reads the same words at the same time
  __shared__ __attribute__((aligned(16))) float wl[kConvSmallMaxMaps * (ROW + 4)];
  const int tid = threadIdx.x;
  const uint32_t p = min(blockIdx.x * CS_THREADS + (uint32_t)tid, total - 1);
  const bool live = blockIdx.x * CS_THREADS + (uint32_t)tid < total;
  const uint32_t mm = (uint32_t)m * m;
  const uint32_t img = fdiv(p, div_mm), pix = p - img * mm;
  const uint32_t y = fdiv(pix, div_m), x = pix - y * m;
  // this lane's source values: requested before the filters are staged, used after
  float patch[DKK];
  const float *src = in + (size_t)img * D * n * n;
#pragma unroll
  for (int c = 0; c < D; ++c)
#pragma unroll
    for (int u = 0; u < KS; ++u)
#pragma unroll
      for (int v = 0; v < KS; ++v) {
        // (an unconditional load from a clamped address, then a select: a conditional load is a branch, and
        // branches serialise the loads' latencies)
        const int sy = (int)y + u - pad, sx = (int)x + v - pad;
        const bool ok = (unsigned)sy < (unsigned)n && (unsigned)sx < (unsigned)n;
        const float val = src[(c * n + min(max(sy, 0), n - 1)) * n + min(max(sx, 0), n - 1)];
        patch[(c * KS + u) * KS + v] = ok ? val : 0.0f;
      }
  for (int e = tid; e < o * (ROW + 4); e += CS_THREADS) {
    const int mo = e / (ROW + 4), j = e - mo * (ROW + 4);
    wl[e] = j < DKK ? w[mo * DKK + j] : (j == ROW && bias) ? bias[mo] : 0.0f;
  }
  __syncthreads();
  if (!live) return;
  float *dst = out + (size_t)img * o * mm + pix;
  for (int mo = 0; mo < o; ++mo) {
    const f4 *wm = reinterpret_cast<const f4 *>(wl + mo * (ROW + 4));
    float s = 0.0f;
#pragma unroll
    for (int q = 0; q < ROW / 4; ++q) {
      const f4 wq = wm[q];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (4 * q + e < DKK) s = __builtin_fmaf(patch[4 * q + e], wq[e], s);
    }
    s += wm[ROW / 4][0];
    dst[(size_t)mo * mm] = (relu && !(s > 0.0f)) ? 0.0f : s;
  }
}

// part[g][mo][j] (j < DKK) and part_bias[g][mo]: the sums over the images of group g.  A workgroup takes MG maps and
// a group of images; its 256 lanes take U pixels of the group each per trip -- a pixel's d*k*k source values are
// loaded once for the MG maps -- with all of a trip's loads requested before its first multiply-add (the kernel is a
// chain of memory latencies otherwise).
template <int KS, int D, int MG, int U>
__global__ __launch_bounds__(CS_THREADS) void conv_small_wgrad_kernel(float *__restrict__ part,
                                                                     float *__restrict__ part_bias,
                                                                     const float *__restrict__ dout,
                                                                     const float *__restrict__ in, int batch, int n,
                                                                     int pad, int o, int m, int imgs_per_group,
                                                                     FastDiv div_mm, FastDiv div_m) {
  constexpr int DKK = ConvSmallShape<KS, D>::DKK, T = CS_THREADS;
  __shared__ float red[T / 64][MG][DKK + 1];
  const int mo0 = blockIdx.x * MG, grp = blockIdx.y, tid = threadIdx.x;
  const uint32_t mm = (uint32_t)m * m;
  const int img0 = grp * imgs_per_group, img1 = min(batch, img0 + imgs_per_group);
  const uint32_t npix = (uint32_t)max(img1 - img0, 0) * mm;
  float acc[MG][DKK], bsum[MG];
#pragma unroll
  for (int g = 0; g < MG; ++g) {
    bsum[g] = 0.0f;
#pragma unroll
    for (int j = 0; j < DKK; ++j) acc[g][j] = 0.0f;
  }
  for (uint32_t p0 = tid; p0 < npix; p0 += T * U) {  // ascending pixels per lane
    float gval[U][MG], xv[U][DKK];
#pragma unroll
    for (int q = 0; q < U; ++q) {
      const uint32_t p = p0 + q * T;
      const bool livep = p < npix;
      const uint32_t pc = livep ? p : 0u;
      const uint32_t li = fdiv(pc, div_mm), pix = pc - li * mm;
      const uint32_t y = fdiv(pix, div_m), x = pix - y * m;
      const uint32_t img = img0 + li;
#pragma unroll
      for (int g = 0; g < MG; ++g) {
        // (unconditional loads from clamped addresses, then selects: a conditional load is a branch, and
        // branches serialise the loads' latencies)
        const float gq = dout[((size_t)img * o + min(mo0 + g, o - 1)) * mm + pix];
        gval[q][g] = (livep && mo0 + g < o) ? gq : 0.0f;
      }
      const float *src = in + (size_t)img * D * n * n;
#pragma unroll
      for (int c = 0; c < D; ++c)
#pragma unroll
        for (int u = 0; u < KS; ++u)
#pragma unroll
          for (int v = 0; v < KS; ++v) {
            const int sy = (int)y + u - pad, sx = (int)x + v - pad;
            const bool ok = (unsigned)sy < (unsigned)n && (unsigned)sx < (unsigned)n;
            const float val = src[(c * n + min(max(sy, 0), n - 1)) * n + min(max(sx, 0), n - 1)];
            xv[q][(c * KS + u) * KS + v] = ok ? val : 0.0f;
          }
    }
#pragma unroll
    for (int q = 0; q < U; ++q)
#pragma unroll
      for (int g = 0; g < MG; ++g) {
        bsum[g] += gval[q][g];
#pragma unroll
        for (int j = 0; j < DKK; ++j) acc[g][j] = __builtin_fmaf(gval[q][g], xv[q][j], acc[g][j]);
      }
  }
  // lane tree within the wavefront, then the wavefronts in order
#pragma unroll
  for (int g = 0; g < MG; ++g)
#pragma unroll
    for (int j = 0; j <= DKK; ++j) {
      const float v = conv_small_wave_sum(j < DKK ? acc[g][j % DKK] : bsum[g]);
      if ((tid & 63) == 63) red[tid >> 6][g][j] = v;
    }
  __syncthreads();
  if (tid < MG * (DKK + 1)) {
    const int g = tid / (DKK + 1), j = tid - g * (DKK + 1), mo = mo0 + g;
    float s = red[0][g][j];
#pragma unroll
    for (int wv = 1; wv < T / 64; ++wv) s += red[wv][g][j];
    if (mo < o) {
      if (j < DKK) part[((size_t)grp * o + mo) * DKK + j] = s;
      else if (part_bias) part_bias[(size_t)grp * o + mo] = s;
    }
  }
}

static bool conv_small_covers(int batch, int d, int n, int ks, int stride, int pad, int o) {
  if (stride != 1 || (ks != 3 && ks != 5) || (d != 1 && d != 3)) return false;
  if (batch <= 0 || n <= 0 || o <= 0 || o > kConvSmallMaxMaps || pad < 0 || pad >= ks) return false;
  const long m = (long)n + 2 * pad - ks + 1;
  if (m <= 0) return false;
  return (double)batch * o * m * m < 1073741824.0 && (double)batch * d * n * n < 1073741824.0;
}

template <int KS, int D>
static int conv_small_forward_launch(float *out, const float *in, const float *w, const float *bias, int batch, int n,
                                     int pad, int o, int relu) {
  const int m = n + 2 * pad - KS + 1;
  const uint32_t total = (uint32_t)batch * m * m;
  hipLaunchKernelGGL((conv_small_forward_kernel<KS, D>), dim3((total + CS_THREADS - 1) / CS_THREADS), dim3(CS_THREADS),
                     0, ctx().stream, out, in, w, bias, n, pad, o, m, total, make_fastdiv((uint32_t)(m * m)),
                     make_fastdiv((uint32_t)m), relu);
  CCT_LAUNCH_CHECK();
  note_kernel("conv_small_forward_kernel<%d,%d>", KS, D);
  return 0;
}

template <int KS, int D>
static int conv_small_wgrad_launch(float *dw, float *db, const float *dout, const float *in, int batch, int n, int pad,
                                   int o) {
  constexpr int DKK = D * KS * KS;
  // maps per workgroup and pixels per lane and trip: what the register file holds (MG * (DKK + 1) sums,
  // U * (DKK + MG) loaded values)
  // (measured on LeNet's first layer: more maps per workgroup save loads but serialise more lane sums per
  // wavefront -- four maps cost 15 us against 12 us for one)
  constexpr int MG = 1, U = DKK <= 27 ? 3 : 1;
  static_assert(MG * (DKK + 1) <= CS_THREADS, "one lane per sum of the workgroup");
  const int m = n + 2 * pad - KS + 1;
  // groups of whole images
  const int map_groups = (o + MG - 1) / MG;
  // (as many as give every lane one trip, up to 64 partial sums for the second launch to add up)
  int groups = (int)(((long)batch * m * m + CS_THREADS * U - 1) / (CS_THREADS * U));
  if (groups > batch) groups = batch;
  if (groups > 64) groups = 64;
  if (groups < 1) groups = 1;
  int per = (batch + groups - 1) / groups;
  groups = (batch + per - 1) / per;
  void *ws = nullptr;
  if (int rc = get_workspace((size_t)groups * o * (DKK + 1) * sizeof(float), &ws)) return rc;
  float *part = (float *)ws, *part_bias = db ? part + (size_t)groups * o * DKK : nullptr;
  hipLaunchKernelGGL((conv_small_wgrad_kernel<KS, D, MG, U>), dim3(map_groups, groups), dim3(CS_THREADS), 0,
                     ctx().stream, part, part_bias, dout, in, batch, n, pad, o, m, per, make_fastdiv((uint32_t)(m * m)),
                     make_fastdiv((uint32_t)m));
  CCT_LAUNCH_CHECK();
  note_kernel("conv_small_wgrad_kernel<%d,%d,%d,%d> groups=%d", KS, D, MG, U, groups);
  return reduce_partial_sums(dw, part, (uint32_t)(o * DKK), db, part_bias, db ? (uint32_t)o : 0u, groups, ctx().stream);
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_conv_small_supported(int batch, int d, int n, int k, int stride, int pad, int o) {
  return conv_small_covers(batch, d, n, k, stride, pad, o) ? 1 : 0;
}

#define CCT_CONV_SMALL_DISPATCH(fn, ...)                           \
  (k == 3 ? (d == 1 ? fn<3, 1>(__VA_ARGS__) : fn<3, 3>(__VA_ARGS__)) \
          : (d == 1 ? fn<5, 1>(__VA_ARGS__) : fn<5, 3>(__VA_ARGS__)))

extern "C" int cct_hip_conv_small_forward(float *out, const float *in, const float *w, const float *bias, int batch,
                                          int d, int n, int k, int pad, int o, int relu) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out && in && w, "conv_small_forward: null argument");
  CCT_REQUIRE(conv_small_covers(batch, d, n, k, 1, pad, o),
              "conv_small_forward: geometry not covered (b=%d d=%d n=%d k=%d pad=%d o=%d)", batch, d, n, k, pad, o);
  return CCT_CONV_SMALL_DISPATCH(conv_small_forward_launch, out, in, w, bias, batch, n, pad, o, relu);
}

extern "C" int cct_hip_conv_small_backward_weights(float *dw, float *db, const float *dout, const float *in, int batch,
                                                   int d, int n, int k, int pad, int o) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dw && dout && in, "conv_small_backward_weights: null argument");
  CCT_REQUIRE(conv_small_covers(batch, d, n, k, 1, pad, o),
              "conv_small_backward_weights: geometry not covered (b=%d d=%d n=%d k=%d pad=%d o=%d)", batch, d, n, k, pad,
              o);
  return CCT_CONV_SMALL_DISPATCH(conv_small_wgrad_launch, dw, db, dout, in, batch, n, pad, o);
}
