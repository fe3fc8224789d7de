// Inverse lowering (col2im lifting) for gfx950, gather formulation, optionally in one launch
// with the bias-gradient reduction.
//
//   dst[ib][id][y][x] = sum over (kr ascending, kc ascending) with cr*s + kr - p == y,
//                       cc*s + kc - p == x, 0 <= cr,cc < m of
//                       src[((id*k + kr)*k + kc) * iB*m*m + ib*m*m + cr*m + cc]
//
// One lane owns one destination pixel and adds its (at most ceil(k/s)^2) contributions in the
// order the reference's scatter loop delivers them (src/sched/DeviceDriver_CPU.cpp:322-345), so
// the result is bit-identical to that loop run on a zero-filled destination.  Every source
// element is read exactly once; lanes of a wave read consecutive addresses of one (kr,kc) plane.
//
// HBM traffic per launch: reads iD*k*k*iB*m*m*4, writes iB*iD*iR*iC*4.  Bound: HBM read bandwidth.
//
// Bias gradient (fused variant): workgroups past the lift range each own one output channel and
// reduce out_grad[b][o][fmap] over b and fmap with per-lane partial sums, a wavefront
// (cross-lane) reduction and a final pass over the workgroup's wave sums.
#include <mutex>

#include "cct_common.h"

namespace cct {

struct LiftParams {
  int m;  // output rows == cols (the reference indexes with oh*cr + cc)
  int k, s, p;
  int iR, iC, iD, iB;
  uint32_t npix;      // iB*iD*iR*iC
  uint32_t nblocks;   // lift workgroups
  uint32_t nbias;     // bias-gradient workgroups; they take the FIRST block ids so that their long
                      // serial reductions start at once and overlap the lift blocks
  size_t plane;       // iB*m*m
  FastDiv div_c, div_r, div_d;
  // bias part: nbias = depth * bsplit workgroups; workgroup (o, s) reduces images
  // [s*bchunk, (s+1)*bchunk) of channel o into partial[o*bsplit + s]; the last one to arrive for a
  // channel adds the partials in ascending s and writes bias_grad[o] (fixed order: deterministic)
  const float *out_grad;
  float *bias_grad;
  float *partial;
  unsigned int *counters;
  int fmap, depth, batch;
  int bsplit, bchunk;
};

constexpr int LIFT_THREADS = 256;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

__device__ void bias_backward_block(const LiftParams &P, int blk) {
  __shared__ float wave_part[LIFT_THREADS / 64];
  __shared__ unsigned int arrived;
  const int tid = threadIdx.x;
  const int o = blk / P.bsplit, sp = blk - o * P.bsplit;
  const int b0 = sp * P.bchunk, b1 = min(P.batch, b0 + P.bchunk);
  // eight images at a time with independent partial sums: eight loads in flight per lane, so the
  // reduction streams at HBM speed next to the gather instead of waiting on one load at a time
  float a[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) a[q] = 0.0f;
  const size_t img = (size_t)P.depth * P.fmap;
  int bi = b0;
  for (; bi + 8 <= b1; bi += 8) {
    const float *g = P.out_grad + ((size_t)bi * P.depth + o) * P.fmap;
    for (int i = tid; i < P.fmap; i += LIFT_THREADS) {
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = g[q * img + i];
#pragma unroll
      for (int q = 0; q < 8; ++q) a[q] += v[q];
    }
  }
  for (; bi < b1; ++bi) {
    const float *g = P.out_grad + ((size_t)bi * P.depth + o) * P.fmap;
    for (int i = tid; i < P.fmap; i += LIFT_THREADS) a[0] += g[i];
  }
  const float a0 = a[0] + a[4], a1 = a[1] + a[5], a2 = a[2] + a[6], a3 = a[3] + a[7];
  float acc = wave_sum((a0 + a1) + (a2 + a3));
  if ((tid & 63) == 0) wave_part[tid >> 6] = acc;
  __syncthreads();
  if (tid == 0) {
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < LIFT_THREADS / 64; ++w) t += wave_part[w];
    if (P.bsplit == 1) {
      P.bias_grad[o] = t;
    } else {
      __hip_atomic_store(&P.partial[blk], t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __threadfence();
      arrived = atomicAdd(&P.counters[o], 1u);
      if (arrived == (unsigned int)P.bsplit - 1) {
        __threadfence();
        float sum = 0.0f;
        for (int q = 0; q < P.bsplit; ++q)
          sum += __hip_atomic_load(&P.partial[o * P.bsplit + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        P.bias_grad[o] = sum;
        P.counters[o] = 0;  // ready for the next launch
      }
    }
  }
}

// Checks the launch just enqueued.  If it was refused while it was meant to use the arrival
// counters, they are flagged so that they are cleared before their next use.
static int check_counter_launch(const LiftParams &P) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  if (P.counters) mark_counters_dirty();
  return set_error((int)e, "lift / bias-gradient launch failed: %s", hipGetErrorString(e));
}

// host side: choose the batch split of the bias reduction (no scratch yet)
static void plan_bias(LiftParams &P, float *bias_grad, const float *out_grad, int fmap, int depth, int batch,
                      bool fused_with_lift) {
  P.out_grad = out_grad; P.bias_grad = bias_grad; P.fmap = fmap; P.depth = depth; P.batch = batch;
  P.partial = nullptr; P.counters = nullptr; P.bsplit = 1; P.bchunk = batch; P.nbias = 0;
  if (!bias_grad) return;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  // alone: two workgroups per CU; next to the lift blocks: about one per CU, so that the reduction
  // streams alongside the gather without crowding it out
  int split = fused_with_lift ? cus / depth : (2 * cus + depth - 1) / depth;
  if (split > batch / 4) split = batch / 4;
  // a channel's whole reduction is a few loads per lane: the split's arrival counter and second pass
  // cost more than they save (LeNet conv2: 10.1 -> 6 us for the fused launch)
  if ((size_t)batch * fmap <= 16384) split = 1;
  if (split < 1 || depth > kMaxCounters) split = 1;
  const int chunk = (batch + split - 1) / split;
  split = (batch + chunk - 1) / chunk;
  P.bsplit = split; P.bchunk = chunk;
  P.nbias = (uint32_t)depth * split;
}

// the same, with the scratch of a split reduction taken from the library's grow-only workspace
static int setup_bias(LiftParams &P, float *bias_grad, const float *out_grad, int fmap, int depth, int batch,
                      bool fused_with_lift) {
  plan_bias(P, bias_grad, out_grad, fmap, depth, batch, fused_with_lift);
  if (P.bsplit > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)depth * P.bsplit * sizeof(float), &ws);
    if (rc) return rc;
    P.partial = (float *)ws;
    rc = get_counters(&P.counters);
    if (rc) return rc;
  }
  return 0;
}

// KT/ST: compile-time kernel size / stride (0 = read from P at run time)
template <int KT, int ST>
__global__ __launch_bounds__(LIFT_THREADS) void lift_kernel(float *__restrict__ dst,
                                                            const float *__restrict__ src,
                                                            const LiftParams P) {
  if (blockIdx.x < P.nbias) {
    bias_backward_block(P, (int)blockIdx.x);
    return;
  }
  const int k = KT ? KT : P.k;
  const int s = ST ? ST : P.s;
  const uint32_t pix = (blockIdx.x - P.nbias) * LIFT_THREADS + threadIdx.x;
  if (pix >= P.npix) return;
  // pix = ((ib*iD + id)*iR + y)*iC + x
  const uint32_t t1 = fdiv(pix, P.div_c);
  const int x = pix - t1 * P.iC;
  const uint32_t t2 = fdiv(t1, P.div_r);
  const int y = t1 - t2 * P.iR;
  const uint32_t ib = fdiv(t2, P.div_d);
  const int id = t2 - ib * P.iD;

  const int m = P.m;
  const float *base = src + (size_t)id * k * k * P.plane + (size_t)ib * m * m;
  float acc = 0.0f;
  const int yp = y + P.p, xp = x + P.p;
  if (ST == 1) {
    // every (kr,kc) is a candidate; out-of-range ones contribute an exact +0
#pragma unroll
    for (int kr = 0; kr < k; ++kr) {
      const int cr = yp - kr;
      const bool rok = (cr >= 0) && (cr < m);
#pragma unroll
      for (int kc = 0; kc < k; ++kc) {
        const int cc = xp - kc;
        const bool ok = rok && (cc >= 0) && (cc < m);
        const size_t off = (size_t)(kr * k + kc) * P.plane + (size_t)(ok ? cr * m + cc : 0);
        const float v = ok ? base[off] : 0.0f;
        acc += v;
      }
    }
  } else {
    for (int kr = yp % s; kr < k; kr += s) {
      const int cr = (yp - kr) / s;
      if (yp < kr) break;
      if (cr >= m) continue;
      for (int kc = xp % s; kc < k; kc += s) {
        const int cc = (xp - kc) / s;
        if (xp < kc) break;
        if (cc >= m) continue;
        acc += base[(size_t)(kr * k + kc) * P.plane + (size_t)(cr * m + cc)];
      }
    }
  }
  dst[pix] = acc;
}

// Strided layers (stride ST > 1): a lane owns ST consecutive destination pixels of a row.  Pixel
// x = ST*l + ph draws on the planes kc == (x + p) mod ST, so for a fixed phase ph the lanes of a
// wavefront read consecutive addresses of ONE (kr, kc) plane -- with one pixel per lane they would
// alternate between ST planes.  Each pixel still adds its terms in (kr, kc) ascending order; the
// ST results leave in one store.
typedef float lift_f4u __attribute__((ext_vector_type(4), aligned(4)));

template <int KT, int ST>
__global__ __launch_bounds__(LIFT_THREADS) void lift_strided_kernel(float *__restrict__ dst,
                                                                    const float *__restrict__ src,
                                                                    const LiftParams P, uint32_t nruns,
                                                                    FastDiv div_runs) {
  if (blockIdx.x < P.nbias) {
    bias_backward_block(P, (int)blockIdx.x);
    return;
  }
  const uint32_t run = (blockIdx.x - P.nbias) * LIFT_THREADS + threadIdx.x;
  if (run >= nruns) return;
  // run = ((ib*iD + id)*iR + y)*runs_per_row + l
  const uint32_t t1 = fdiv(run, div_runs);
  const int l = run - t1 * div_runs.div;
  const uint32_t t2 = fdiv(t1, P.div_r);
  const int y = t1 - t2 * P.iR;
  const uint32_t ib = fdiv(t2, P.div_d);
  const int id = t2 - ib * P.iD;
  const int m = P.m;
  const float *base = src + (size_t)id * KT * KT * P.plane + (size_t)ib * m * m;
  const int yp = y + P.p;
  // every candidate (jr, jc) is loaded from a clamped address without a branch, so all loads of a
  // lane are in flight together; candidates outside the kernel or the output contribute an exact +0
  constexpr int NJ = (KT + ST - 1) / ST;
  float acc[ST];
#pragma unroll
  for (int ph = 0; ph < ST; ++ph) {
    const int xp = l * ST + ph + P.p;
    float v[NJ][NJ];
#pragma unroll
    for (int jr = 0; jr < NJ; ++jr) {
      const int kr = yp % ST + jr * ST, cr = (yp - kr) / ST;  // yp - kr is a multiple of ST
      const bool rok = kr < KT && yp >= kr && cr < m;
#pragma unroll
      for (int jc = 0; jc < NJ; ++jc) {
        const int kc = xp % ST + jc * ST, cc = (xp - kc) / ST;
        const bool ok = rok && kc < KT && xp >= kc && cc < m;
        const size_t off = ok ? (size_t)(kr * KT + kc) * P.plane + (size_t)(cr * m + cc) : 0;
        const float t = base[off];
        v[jr][jc] = ok ? t : 0.0f;
      }
    }
    float a = 0.0f;
#pragma unroll
    for (int jr = 0; jr < NJ; ++jr)
#pragma unroll
      for (int jc = 0; jc < NJ; ++jc) a += v[jr][jc];
    acc[ph] = a;
  }
  float *out = dst + (size_t)t1 * P.iC + (size_t)l * ST;
  const int n = min(ST, P.iC - l * ST);
  if (ST == 4 && n == 4) {
    const lift_f4u v = {acc[0], acc[1], acc[2], acc[3]};
    *reinterpret_cast<lift_f4u *>(out) = v;
  } else {
#pragma unroll
    for (int ph = 0; ph < ST; ++ph)
      if (ph < n) out[ph] = acc[ph];
  }
}

static int launch_lift(float *dst, const float *src, const cct_inverse_lower_cube_args *a,
                       float *bias_grad, const float *out_grad, int fmap, int depth, int batch) {
  CCT_REQUIRE(dst && src && a, "inverse_lower_cube: null argument");
  CCT_REQUIRE(a->data_output_width == a->data_output_height,
              "inverse_lower_cube: output must be square (%zu x %zu)", a->data_output_width,
              a->data_output_height);
  CCT_REQUIRE(a->stride >= 1 && a->kernel_size >= 1, "inverse_lower_cube: bad kernel/stride");
  const size_t npix = a->iB * a->iD * a->iR * a->iC;
  const size_t m = a->data_output_width;
  CCT_REQUIRE(npix < (1ull << 31) && a->iB * m * m < (1ull << 31),
              "inverse_lower_cube: tensor too large for 31-bit position arithmetic");
  LiftParams P;
  P.m = (int)m; P.k = (int)a->kernel_size; P.s = (int)a->stride; P.p = (int)a->padding;
  P.iR = (int)a->iR; P.iC = (int)a->iC; P.iD = (int)a->iD; P.iB = (int)a->iB;
  P.npix = (uint32_t)npix;
  P.nblocks = (uint32_t)((npix + LIFT_THREADS - 1) / LIFT_THREADS);
  P.plane = a->iB * m * m;
  P.div_c = make_fastdiv(P.iC); P.div_r = make_fastdiv(P.iR); P.div_d = make_fastdiv(P.iD);
  int rc = setup_bias(P, bias_grad, out_grad, fmap, depth, batch, true);
  if (rc) return rc;
  const uint32_t grid = P.nblocks + P.nbias;
  if (grid == 0) return 0;
  hipStream_t st = ctx().stream;
  if (P.k == 5 && P.s == 1) {
    hipLaunchKernelGGL((lift_kernel<5, 1>), dim3(grid), dim3(LIFT_THREADS), 0, st, dst, src, P);
    note_kernel("lift_kernel<5,1> bias_blocks=%u", P.nbias);
  } else if (P.k == 3 && P.s == 1) {
    hipLaunchKernelGGL((lift_kernel<3, 1>), dim3(grid), dim3(LIFT_THREADS), 0, st, dst, src, P);
    note_kernel("lift_kernel<3,1> bias_blocks=%u", P.nbias);
  } else if (P.k == 11 && P.s == 4) {
    const uint32_t per_row = (uint32_t)((P.iC + 3) / 4);
    const size_t nruns = (size_t)P.iB * P.iD * P.iR * per_row;
    const uint32_t blocks = (uint32_t)((nruns + LIFT_THREADS - 1) / LIFT_THREADS);
    hipLaunchKernelGGL((lift_strided_kernel<11, 4>), dim3(blocks + P.nbias), dim3(LIFT_THREADS), 0, st, dst, src, P,
                       (uint32_t)nruns, make_fastdiv(per_row));
    note_kernel("lift_strided_kernel<11,4> bias_blocks=%u", P.nbias);
  } else {
    hipLaunchKernelGGL((lift_kernel<0, 0>), dim3(grid), dim3(LIFT_THREADS), 0, st, dst, src, P);
    note_kernel("lift_kernel<0,0> bias_blocks=%u", P.nbias);
  }
  return check_counter_launch(P);
}

}  // namespace cct

using namespace cct;

// ---- scratch of the entry point that allocates nothing ------------------------------------------
// Arrival counters (one per channel) followed by the partial sums of a split reduction.  Every GPU
// the library runs on holds its own copy of this array until the process ends.
constexpr int kNoAllocMaxDepth = 4096;       // channels
constexpr int kNoAllocMaxPartials = 16384;   // depth * batch split
constexpr size_t kNoAllocCounterBytes = (size_t)kNoAllocMaxDepth * sizeof(unsigned int);
constexpr size_t kNoAllocScratchBytes = kNoAllocCounterBytes + (size_t)kNoAllocMaxPartials * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// The array's name is only a host-side stand-in: its device address differs per GPU and comes from
// hipGetSymbolAddress, asked once per device with that device current.
constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mu;

static int scratch_address(void **out) {
  const int dev = ctx().device;
  CCT_REQUIRE(dev >= 0 && dev < kMaxDevices, "backward_bias_noalloc: device %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    CCT_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    CCT_REQUIRE(ptr != nullptr, "backward_bias_noalloc: no device address for the scratch array");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

__global__ void zero_words_kernel(unsigned int *__restrict__ p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

extern "C" int cct_hip_inverse_lower_cube(float *dst, const float *src,
                                          const cct_inverse_lower_cube_args *args) {
  CCT_ENSURE_INIT();
  return launch_lift(dst, src, args, nullptr, nullptr, 0, 0, 0);
}

extern "C" int cct_hip_inverse_lower_cube_bias_backward(float *dst, const float *src,
                                                        const cct_inverse_lower_cube_args *args,
                                                        float *bias_grad, const float *out_grad,
                                                        int fmap_size, int depth, int batch_size) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(bias_grad && out_grad, "inverse_lower_cube_bias_backward: null bias argument");
  CCT_REQUIRE(fmap_size > 0 && depth > 0 && batch_size > 0,
              "inverse_lower_cube_bias_backward: fmap/depth/batch must be positive");
  return launch_lift(dst, src, args, bias_grad, out_grad, fmap_size, depth, batch_size);
}

extern "C" int cct_hip_backward_bias(float *bias_grad, const float *out_grad, int fmap_size,
                                     int depth, int batch_size) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(bias_grad && out_grad, "backward_bias: null argument");
  CCT_REQUIRE(fmap_size > 0 && depth > 0 && batch_size > 0,
              "backward_bias: fmap/depth/batch must be positive");
  // the same kernel with zero lift blocks
  LiftParams P = {};
  P.nblocks = 0;
  int rc = setup_bias(P, bias_grad, out_grad, fmap_size, depth, batch_size, false);
  if (rc) return rc;
  hipLaunchKernelGGL((lift_kernel<0, 0>), dim3(P.nbias), dim3(LIFT_THREADS), 0, ctx().stream,
                     (float *)nullptr, (const float *)nullptr, P);
  return check_counter_launch(P);
}

extern "C" int cct_hip_backward_bias_noalloc(float *bias_grad, const float *out_grad, int fmap_size,
                                             int depth, int batch_size) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(bias_grad && out_grad, "backward_bias_noalloc: null argument");
  CCT_REQUIRE(fmap_size > 0 && depth > 0 && batch_size > 0,
              "backward_bias_noalloc: fmap/depth/batch must be positive");
  CCT_REQUIRE(depth <= kNoAllocMaxDepth,
              "backward_bias_noalloc: depth %d exceeds the built-in scratch (at most %d channels); "
              "use cct_hip_backward_bias",
              depth, kNoAllocMaxDepth);
  LiftParams P = {};
  P.nblocks = 0;
  plan_bias(P, bias_grad, out_grad, fmap_size, depth, batch_size, false);
  CCT_REQUIRE((long)depth * P.bsplit <= kNoAllocMaxPartials,
              "backward_bias_noalloc: %d x %d partial sums exceed the built-in scratch (at most %d); "
              "use cct_hip_backward_bias",
              depth, P.bsplit, kNoAllocMaxPartials);
  hipStream_t st = ctx().stream;
  if (P.bsplit > 1) {
    void *base = nullptr;
    int rc = scratch_address(&base);
    if (rc) return rc;
    P.counters = (unsigned int *)base;
    P.partial = (float *)((unsigned char *)base + kNoAllocCounterBytes);
    // the array keeps the last call's contents: the counters this launch uses must start at zero
    // (a fill kernel, not a memset node, so that a caller may capture the call into a graph)
    hipLaunchKernelGGL(zero_words_kernel, dim3((depth + 255) / 256), dim3(256), 0, st, P.counters, depth);
    CCT_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL((lift_kernel<0, 0>), dim3(P.nbias), dim3(LIFT_THREADS), 0, st, (float *)nullptr,
                     (const float *)nullptr, P);
  CCT_LAUNCH_CHECK();
  return 0;
}
