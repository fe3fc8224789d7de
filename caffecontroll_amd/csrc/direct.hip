// Stride-1 convolution as a direct contraction on the gfx950 matrix cores, without the lowered
// matrix in memory.
//
//   dst[img][m][y][x] = bias[m] + sum_{c,u,v} wt[c][m][u*KS+v] * src[img][c][y-pad+u][x-pad+v]
//
// (out-of-image source elements count as zero; dst is ho x ho with ho = hs + 2*pad - KS + 1).
// Two uses, both of which replace a chain of the lowering pipeline:
//   * forward:        wt = model transposed to [d][o][k*k], src = input, pad = p
//                     (lower_cube + forward GEMM + output remap + bias)
//   * data gradient:  wt = model [o][d][k*k] with every k x k filter reversed, src = output
//                     gradient, pad = k-1-p   (gradient remap + data-gradient GEMM + lifting)
// The sums run over (c,u,v) in a different order than the lowered GEMM, so results agree with
// the lowering path to fp32 rounding, not bit for bit.
//
// One workgroup (4 wavefronts) computes BM = 32*TMB output maps x BN = 128*TNB consecutive output
// pixels (pixels are numbered across the whole batch, so a tile may straddle images).  The
// contraction index is consumed two*CP channels per step:
//   * the weight slab of a channel, wt[c][m0..m0+BM)[KS*KS], is one contiguous run in memory and is
//     copied to LDS as is (16-byte loads);
//   * the source rows that the tile's pixels touch are copied to a zero-bordered LDS patch of
//     PW-float rows ("row v" of the patch = row v of the virtual stack of zero-padded images);
//     border elements are cleared once and never written, so padding costs nothing per step;
//   * MFMA v_mfma_f32_32x32x2_f32 takes k = (channel 2cp, tap j) from lanes 0-31 and
//     k = (channel 2cp+1, tap j) from lanes 32-63, so every fragment is one ds_read_b32 at
//     lane base + compile-time offset: no address arithmetic inside the loop.
// Two LDS stages, one barrier per step; the global loads of step t+1 are in flight during the
// MFMAs of step t.
//
// Bound: fp32 MFMA rate.  Algorithmic work 2 * mtot * batch*ho*ho * kc*KS*KS FLOP per call.
#include <cstdlib>

#include "cct_common.h"

namespace cct {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));

struct DirectArgs {
  const float *wt;    // slab buffer [kc padded to 4][mtot padded to whole tiles][KS*KS], zero padding
  const float *src;   // [batch][kc][hs][hs]
  float *dst;         // [batch][mtot][ho][ho]
  const float *bias;  // [mtot] or null
  int batch, kc, mtot, hs, ho, pad;
  int hp;             // ho + KS - 1 = hs + 2*pad: rows (and columns) of a zero-padded source image
  int pr;             // patch rows per channel
  int nsteps;         // ceil(kc / channels per step)
  int slab_stride;    // floats between channels of the slab buffer (padded map count * KS*KS)
  uint32_t ptot;      // batch * ho * ho
  uint32_t tiles_m, ntiles;
  FastDiv div_ho, div_ho2, div_hp, div_pr;
};

constexpr int kDirectPatchLoads = 8;  // source elements per lane per step, at most

// global -> LDS without passing through registers.  `lds_wave_base` is the wave-uniform LDS address
// that lane 0's data goes to; lane l's 16 (or 4) bytes land 16*l (4*l) bytes further on.
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;
__device__ __forceinline__ void lds_dma16(const float *g, float *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(uintptr_t)lds_wave_base, 16, 0, 0);
}
__device__ __forceinline__ void lds_dma4(const float *g, float *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(uintptr_t)lds_wave_base, 4, 0, 0);
}
// all of this wave's global->LDS loads have landed (vmcnt(0); expcnt/lgkmcnt left alone)
__device__ __forceinline__ void lds_dma_wait() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Fragments of contraction index idx = cp*KS*KS + j (idx is a constant after unrolling): weights of
// tap j of channel pair cp for TMB row blocks, source elements under tap j for TNB pixel blocks.
template <int KS, int TMB, int TNB, int PW>
__device__ __forceinline__ void direct_frags(float (&fa)[TMB], float (&fb)[TNB], const float *__restrict__ sm,
                                             int abase, const int (&bbase)[TNB], int pair_stride, int idx) {
  constexpr int KK = KS * KS, BM = 32 * TMB;
  const int cp = idx / KK, j = idx % KK, u = j / KS, v = j % KS;
#pragma unroll
  for (int a = 0; a < TMB; ++a) fa[a] = sm[abase + cp * (2 * BM * KK) + a * (32 * KK) + j];
#pragma unroll
  for (int b = 0; b < TNB; ++b) fb[b] = sm[bbase[b] + cp * pair_stride + u * PW + v];
}

template <int KS, int TMB, int TNB, int CP, int PW>
__global__ __launch_bounds__(256, 2) void conv_direct_kernel(const DirectArgs g) {
  constexpr int KK = KS * KS, BM = 32 * TMB, BN = 128 * TNB, NC = 2 * CP;
  constexpr int ASZ = NC * BM * KK;           // floats of weight slabs per stage
  constexpr int SLAB4 = BM * KK / 4;          // 16-byte vectors per slab
  constexpr int NA4 = (ASZ / 4 + 255) / 256;  // 16-byte vectors per lane per stage
  constexpr int NPL = kDirectPatchLoads;
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int psz = NC * g.pr * PW;  // floats of patches per stage
  const int stage = ASZ + psz;     // multiple of 4: PW is

  const uint32_t id = xcd_remap(blockIdx.x, g.ntiles);
  const uint32_t tn = id / g.tiles_m, tm = id - tn * g.tiles_m;
  const int m0 = tm * BM;
  const uint32_t p0 = tn * BN;
  const int ho2 = g.ho * g.ho;

  // first patch row: the virtual row of the tile's first pixel
  const uint32_t img0 = fdiv(p0, g.div_ho2);
  const uint32_t y0 = fdiv(p0 - img0 * ho2, g.div_ho);
  const int v_lo = img0 * g.hp + y0;

  // ---- per-lane loader state -------------------------------------------------------------
  // Operands go from global memory straight into LDS (global_load_lds): a wave's load writes its
  // 64 lanes' data to consecutive LDS addresses, so LDS element e is fetched by lane e % 64 of the
  // wave-instruction that covers e.  Every address is a wave-uniform base that advances per step
  // plus a per-lane offset fixed for the whole tile.
  //   weights: the slab buffer is padded with zero rows and zero channels up to whole tiles and
  //            whole steps, so the loads need no bounds tests;
  //   source : patch element e = (channel c, patch row, patch column); elements outside the image
  //            are never loaded -- their LDS words are cleared once below and stay zero.  A
  //            channel past the last one (final step only) is not loaded either: whatever the
  //            patch holds there is finite and meets zero weights.
  uint32_t aoff[NA4];
#pragma unroll
  for (int i = 0; i < NA4; ++i) {
    const int e4 = tid + i * 256;
    const int c = e4 / SLAB4, f = (e4 - c * SLAB4) * 4;
    aoff[i] = (uint32_t)(c * g.slab_stride + f);
  }
  uint32_t psrc[NPL];
  uint32_t mask_all = 0, mask_last = 0;  // bit i: element i is loaded (any step / final step)
  const int last_channels = g.kc - (g.nsteps - 1) * NC;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const uint32_t e = tid + i * 256;
    const uint32_t pc = e % PW, rest = e / PW;
    const uint32_t c = fdiv(rest, g.div_pr), prow = rest - c * g.pr;
    const uint32_t v = v_lo + prow;
    const uint32_t img = fdiv(v, g.div_hp);
    const int srow = (int)(v - img * g.hp) - g.pad, scol = (int)pc - g.pad;
    const bool ok = c < (uint32_t)NC && img < (uint32_t)g.batch && (unsigned)srow < (unsigned)g.hs &&
                    (unsigned)scol < (unsigned)g.hs;
    psrc[i] = ok ? ((img * g.kc + c) * g.hs + srow) * g.hs + scol : 0u;
    mask_all |= (ok ? 1u : 0u) << i;
    mask_last |= ((ok && (int)c < last_channels) ? 1u : 0u) << i;
  }
  const size_t a_step = (size_t)NC * g.slab_stride, b_step = (size_t)NC * g.hs * g.hs;
  const float *a_tile = g.wt + (size_t)m0 * KK;
  const int wave_elem0 = wave * 64;  // first element of this wave within a 256-element pass

// global -> LDS stage s for step t (asynchronous; completion = vmcnt)
#define CCT_DIRECT_ISSUE(t, s)                                                                 \
  do {                                                                                         \
    float *st_ = smem + (s) * stage;                                                           \
    const float *ga_ = a_tile + (size_t)(t) * a_step;                                          \
    _Pragma("unroll") for (int i = 0; i < NA4; ++i) {                                          \
      if ((i + 1) * 256 <= ASZ / 4 || tid + i * 256 < ASZ / 4)                                 \
        lds_dma16(ga_ + aoff[i], st_ + (i * 256 + wave_elem0) * 4);                            \
    }                                                                                          \
    const float *gb_ = g.src + (size_t)(t) * b_step;                                           \
    const uint32_t bm_ = ((t) == g.nsteps - 1) ? mask_last : mask_all;                         \
    _Pragma("unroll") for (int i = 0; i < NPL; ++i) {                                          \
      if ((bm_ >> i) & 1u) lds_dma4(gb_ + psrc[i], st_ + ASZ + i * 256 + wave_elem0);          \
    }                                                                                          \
  } while (0)

  // clear the patches of both stages once: borders and rows outside the images stay zero
  for (int s2 = 0; s2 < 2; ++s2)
    for (int e = tid; e < psz; e += 256) smem[s2 * stage + ASZ + e] = 0.f;
  __syncthreads();

  // ---- per-lane fragment bases --------------------------------------------------------------
  const int abase = h * (BM * KK) + r * KK;
  int bbase[TNB];
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    uint32_t p = p0 + wave * (32 * TNB) + b * 32 + r;
    p = min(p, g.ptot - 1);
    const uint32_t img = fdiv(p, g.div_ho2);
    const uint32_t pix = p - img * ho2;
    const uint32_t y = fdiv(pix, g.div_ho), x = pix - y * g.ho;
    bbase[b] = ASZ + h * (g.pr * PW) + (int)(img * g.hp + y - v_lo) * PW + (int)x;
  }
  const int pair_stride = 2 * g.pr * PW;  // patch floats per channel pair

  v16f acc[TMB][TNB];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int b = 0; b < TNB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.0f;

  CCT_DIRECT_ISSUE(0, 0);
  lds_dma_wait();
  __syncthreads();

  for (int t = 0; t < g.nsteps; ++t) {
    const float *sm = smem + (t & 1) * stage;
    // every wave finished reading the other stage before the barrier that ended step t-1
    if (t + 1 < g.nsteps) CCT_DIRECT_ISSUE(t + 1, (t & 1) ^ 1);
    // Contraction indices are taken two at a time (neighbouring taps sit in neighbouring LDS words,
    // which lets the compiler fetch both with one ds_read2); the fragments of pair q+1 are
    // requested before the MFMAs of pair q.
    constexpr int NI = CP * KK, NQ = (NI + 1) / 2;
    float fa[2][2][TMB], fb[2][2][TNB];
    direct_frags<KS, TMB, TNB, PW>(fa[0][0], fb[0][0], sm, abase, bbase, pair_stride, 0);
    if (NI > 1) direct_frags<KS, TMB, TNB, PW>(fa[0][1], fb[0][1], sm, abase, bbase, pair_stride, 1);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int nb = (q + 1) & 1, cb = q & 1;
      if (2 * q + 2 < NI)
        direct_frags<KS, TMB, TNB, PW>(fa[nb][0], fb[nb][0], sm, abase, bbase, pair_stride, 2 * q + 2);
      if (2 * q + 3 < NI)
        direct_frags<KS, TMB, TNB, PW>(fa[nb][1], fb[nb][1], sm, abase, bbase, pair_stride, 2 * q + 3);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (2 * q + e < NI) {
#pragma unroll
          for (int a2 = 0; a2 < TMB; ++a2)
#pragma unroll
            for (int b2 = 0; b2 < TNB; ++b2)
              acc[a2][b2] =
                  __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][e][a2], fb[cb][e][b2], acc[a2][b2], 0, 0, 0);
        }
      }
      // Issue order inside this pair: one LDS read (of the next pair's fragments) after every few
      // MFMAs, so the reads are in flight a whole pair ahead of their use and the matrix pipe never
      // waits on LDS latency; the fence keeps the next pair's instructions from drifting up.
      {
        constexpr int NR = TMB + TNB, NM = 2 * TMB * TNB, PER = NM / (NR + 1) > 0 ? NM / (NR + 1) : 1;
#pragma unroll
        for (int k2 = 0; k2 < NR; ++k2) {
          __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NM - NR * PER > 0 ? NM - NR * PER : 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    lds_dma_wait();
    __syncthreads();
  }
#undef CCT_DIRECT_ISSUE

  // ---- epilogue: accumulator register v of lane (r,h) is row 8*(v/4) + 4*h + v%4, column r ----
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    const uint32_t p = p0 + wave * (32 * TNB) + b * 32 + r;
    if (p >= g.ptot) continue;
    const uint32_t img = fdiv(p, g.div_ho2);
    float *out = g.dst + (size_t)img * g.mtot * ho2 + (p - img * ho2);
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < g.mtot) out[(size_t)row * ho2] = acc[a][b][v] + (g.bias ? g.bias[row] : 0.f);
      }
  }
}

// Output-map tile (in 32-row blocks) for `mtot` maps: least padding, larger tile on ties.
static int direct_tmb(int mtot) {
  int tmb = 4;
  long best = -1;
  for (int cand = 4; cand >= 2; --cand) {
    const long padded = (long)((mtot + 32 * cand - 1) / (32 * cand)) * 32 * cand;
    if (best < 0 || padded < best) { best = padded; tmb = cand; }
  }
  return tmb;
}
// Slab buffer dimensions: maps padded to whole tiles, channels to a multiple of 4 (a whole step).
static int direct_padded_maps(int mtot) {
  const int bm = 32 * direct_tmb(mtot);
  return (mtot + bm - 1) / bm * bm;
}
static int direct_padded_channels(int kc) { return (kc + 3) / 4 * 4; }

// wt[c][m][j] = w[m][c][j] (forward slabs) or w[c][m][KK-1-j] (data-gradient slabs: every filter
// reversed), zero for padding maps and channels.  `n_c`, `n_m` are the real slab dimensions,
// `p_m` the padded map count; one thread per element of the padded buffer.
__global__ __launch_bounds__(256) void direct_slab_kernel(float *__restrict__ wt, const float *__restrict__ w,
                                                          int n_c, int n_m, int p_m, uint32_t total, int kk,
                                                          int reversed, FastDiv div_kk, FastDiv div_m) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const uint32_t cm = fdiv(e, div_kk), j = e - cm * kk;
  const uint32_t c = fdiv(cm, div_m), m = cm - c * p_m;
  float v = 0.f;
  if (c < (uint32_t)n_c && m < (uint32_t)n_m)
    v = reversed ? w[((size_t)c * n_m + m) * kk + (kk - 1 - j)] : w[((size_t)m * n_c + c) * kk + j];
  wt[e] = v;
}

struct DirectPlan {
  int ks, tmb, tnb, cp, pw, pr;
  size_t lds;
};

// Chooses the kernel instance for a geometry; returns false when the direct path does not cover it.
static bool direct_plan(int batch, int kc, int mtot, int hs, int ks, int pad, DirectPlan *pl) {
  if (ks != 3 && ks != 5) return false;
  if (pad < 0 || pad > ks - 1 || batch <= 0 || kc <= 0 || mtot <= 0) return false;
  const int ho = hs + 2 * pad - ks + 1, hp = ho + ks - 1;
  if (ho <= 0) return false;
  const int pw = hp <= 16 ? 16 : 32;
  if (hp > pw) return false;
  if ((double)batch * kc * hs * hs >= 2147483648.0 || (double)batch * ho * ho >= 2147483648.0) return false;
  const int cp = ks == 3 ? 2 : 1;
  const int tmb = direct_tmb(mtot);
  const long tiles_m = (mtot + 32 * tmb - 1) / (32 * tmb);
  const long ptot = (long)batch * ho * ho;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  for (int tnb = 2; tnb >= 1; --tnb) {
    const int bn = 128 * tnb;
    const int rows = (ho - 1 + bn - 1) / ho + 1, imgs = (ho * ho - 1 + bn - 1) / (ho * ho) + 1;
    const int pr = rows - 1 + (imgs - 1) * (ks - 1) + ks;
    const long patch = 2L * cp * pr * pw;
    const size_t lds = 2 * (size_t)(2 * cp * 32 * tmb * ks * ks + patch) * sizeof(float);
    const long tiles = tiles_m * ((ptot + bn - 1) / bn);
    const bool fits = patch <= 256L * kDirectPatchLoads && lds <= 64 * 1024;
    // the wide tile only when it still gives every compute unit several workgroups
    if (fits && (tnb == 1 || tiles >= 4L * cus)) {
      pl->ks = ks; pl->tmb = tmb; pl->tnb = tnb; pl->cp = cp; pl->pw = pw; pl->pr = pr; pl->lds = lds;
      return true;
    }
  }
  return false;
}

template <int KS, int CP, int PW>
static int direct_launch_ks(const DirectArgs &g, const DirectPlan &pl, hipStream_t st) {
  dim3 grid(g.ntiles), block(256);
#define CCT_DIRECT_CASE(TMB, TNB)                                                                      \
  if (pl.tmb == TMB && pl.tnb == TNB) {                                                                \
    hipLaunchKernelGGL((conv_direct_kernel<KS, TMB, TNB, CP, PW>), grid, block, pl.lds, st, g);        \
    CCT_LAUNCH_CHECK();                                                                                \
    return 0;                                                                                          \
  }
  CCT_DIRECT_CASE(2, 1) CCT_DIRECT_CASE(3, 1) CCT_DIRECT_CASE(4, 1)
  CCT_DIRECT_CASE(2, 2) CCT_DIRECT_CASE(3, 2) CCT_DIRECT_CASE(4, 2)
#undef CCT_DIRECT_CASE
  return set_error(CCT_HIP_EINVAL, "conv_direct: no kernel instance for tile %dx%d", pl.tmb, pl.tnb);
}

static int conv_direct(const float *wt, const float *src, float *dst, const float *bias, int batch, int kc,
                       int mtot, int hs, int ks, int pad) {
  DirectPlan pl;
  CCT_REQUIRE(direct_plan(batch, kc, mtot, hs, ks, pad, &pl),
              "conv_direct: geometry not covered (k=%d pad=%d size=%d)", ks, pad, hs);
  DirectArgs g;
  g.wt = wt; g.src = src; g.dst = dst; g.bias = bias;
  g.batch = batch; g.kc = kc; g.mtot = mtot; g.hs = hs; g.pad = pad;
  g.ho = hs + 2 * pad - ks + 1;
  g.hp = g.ho + ks - 1;
  g.pr = pl.pr;
  g.nsteps = (kc + 2 * pl.cp - 1) / (2 * pl.cp);
  CCT_REQUIRE((uintptr_t)wt % 16 == 0, "conv_direct: slab buffer must be 16-byte aligned");
  g.slab_stride = direct_padded_maps(mtot) * ks * ks;
  g.ptot = (uint32_t)((long)batch * g.ho * g.ho);
  g.tiles_m = (uint32_t)((mtot + 32 * pl.tmb - 1) / (32 * pl.tmb));
  const uint32_t bn = 128 * pl.tnb;
  g.ntiles = g.tiles_m * ((g.ptot + bn - 1) / bn);
  g.div_ho = make_fastdiv((uint32_t)g.ho);
  g.div_ho2 = make_fastdiv((uint32_t)(g.ho * g.ho));
  g.div_hp = make_fastdiv((uint32_t)g.hp);
  g.div_pr = make_fastdiv((uint32_t)g.pr);
  hipStream_t st = ctx().stream;
  if (ks == 5) return pl.pw == 16 ? direct_launch_ks<5, 1, 16>(g, pl, st) : direct_launch_ks<5, 1, 32>(g, pl, st);
  return pl.pw == 16 ? direct_launch_ks<3, 2, 16>(g, pl, st) : direct_launch_ks<3, 2, 32>(g, pl, st);
}


// ---------------------------------------------------------------------------------------------
// Weight gradient without the lowered matrix:
//   dW[oo][c][kr][kc] = sum_{img,r,x} dout[img][oo][r][x] * src[img][c][r-pad+kr][x-pad+kc]
// as a GEMM with M = output maps, N = (c,kr,kc) columns and the contraction over output pixels.
// A workgroup owns BM x BN of dW and a range of contraction steps; one step is two output rows
// (r0, r0+1) of one image: MFMA lanes 0-31 take pixel (r0, x), lanes 32-63 pixel (r0+1, x).  Per
// step the workgroup stages dout[img][m0..m0+BM)[rows r0,r0+1] (row stride odd: conflict-free
// fragment reads) and, for the channels its columns touch, the KS+1 zero-padded source rows
// under those two output rows; each lane's fragment addresses are base + x, so the loop over x
// only bumps two offsets.  Single LDS stage with the next step's global loads parked in
// registers during the MFMAs.  Partial sums of the step ranges go to a workspace and are added in
// a fixed order by direct_reduce_kernel (run-to-run identical results).
struct WgradArgs {
  const float *dout;  // [batch][o][ho][ho]
  const float *src;   // [batch][d][hs][hs]
  float *out;         // [splits][o][ncols]
  int batch, o, d, hs, ho, pad;
  int ncols;          // d * KS * KS
  int chunks;         // row pairs per image: ceil(ho / 2)
  int ast;            // floats between rows of the staged dout slab (odd)
  int steps_total, steps_per_split;
  uint32_t tiles_m, tiles_n, ntiles, nblocks;
  FastDiv div_chunks;
};

template <int KS, int PW>
struct WgradStrides {
  static constexpr int PWS = PW + ((KS - PW) % 32 + 32) % 32;                 // >= PW, == KS (mod 32)
  static constexpr int RAW = (KS + 1) * PWS;
  static constexpr int PCH = RAW + ((KS * KS - RAW) % 32 + 32) % 32;          // >= RAW, == KS*KS (mod 32)
};

template <int KS, int TMB, int TNB, int PW>
__global__ __launch_bounds__(256, 2) void conv_direct_wgrad_kernel(const WgradArgs g) {
  constexpr int KK = KS * KS, BM = 32 * TMB, BN = 128 * TNB;
  constexpr int PRW = KS + 1;                   // patch rows per channel
  // LDS strides of the patch.  A wave's 32 columns are consecutive (c,kr,kc) triples that read
  // patch offset c*PCH + kr*PWS + kc + x: with PWS = KS and PCH = KS*KS (mod 32) that offset is the
  // column number plus a constant, i.e. 32 different banks.
  constexpr int PWS = WgradStrides<KS, PW>::PWS, PCH = WgradStrides<KS, PW>::PCH;
  constexpr int NCH = (BN - 1) / KK + 2;        // channels a column tile can touch
  constexpr int NAL = BM / 4;                   // dout loads per lane per step (4 maps per pass)
  constexpr int RPP = 256 / PW;                 // patch rows per pass
  constexpr int CPP = RPP / PRW;                // whole channels per pass
  constexpr int NBL = (NCH + CPP - 1) / CPP;    // source loads per lane per step
  static_assert(CPP >= 1, "a pass must hold one channel's patch rows");
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float *sa = smem;
  float *sb = smem + ((BM * g.ast + 3) & ~3);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t z = flat / g.ntiles, id = flat - z * g.ntiles;
  const uint32_t tm = id / g.tiles_n, tn = id - tm * g.tiles_n;  // column tiles of one row tile run together
  const int m0 = tm * BM, n0 = tn * BN, ch0 = n0 / KK;
  const int s_beg = z * g.steps_per_split, s_end = min(g.steps_total, s_beg + g.steps_per_split);
  const int ho2 = g.ho * g.ho, hs2 = g.hs * g.hs;

  // Loaders.  Every load address is a wave-uniform base (image, pass) plus a per-lane offset that
  // does not change between steps.
  //   dout: lane -> staged column ai (two output rows side by side), map arow + 4*pass
  //   src : lane -> patch column pcol, patch row prow of channel chsub + CPP*pass
  const int ai = tid & 63, arow = tid >> 6;
  const bool a_ok = ai < 2 * g.ho;
  const int a_lane = arow * ho2 + ai;
  const int pcol = tid % PW, q = tid / PW;
  const int chsub = q / PRW, prow = q - chsub * PRW;
  const int scol = pcol - g.pad;
  const bool b_lane_ok = chsub < CPP && (unsigned)scol < (unsigned)g.hs;
  const int b_lane = chsub * hs2 + prow * g.hs + scol;
  const int sb_lane = chsub * PCH + prow * PWS + pcol;

  float ra[NAL], rb[NBL];
#define CCT_WGRAD_FETCH(s)                                                                        \
  do {                                                                                            \
    const uint32_t img_ = fdiv((uint32_t)(s), g.div_chunks);                                      \
    const int r0_ = 2 * ((s) - (int)img_ * g.chunks);                                             \
    const bool pok_ = a_ok && r0_ * g.ho + ai < ho2;                                              \
    const float *pa_ = g.dout + ((size_t)img_ * g.o + m0) * ho2 + r0_ * g.ho;                     \
    _Pragma("unroll") for (int k = 0; k < NAL; ++k) {                                             \
      ra[k] = (pok_ && m0 + arow + 4 * k < g.o) ? (pa_ + (size_t)k * 4 * ho2)[a_lane] : 0.f;      \
    }                                                                                             \
    const bool rok_ = b_lane_ok && (unsigned)(r0_ + prow - g.pad) < (unsigned)g.hs;               \
    const float *pb_ = g.src + ((size_t)img_ * g.d + ch0) * hs2 + (r0_ - g.pad) * g.hs;           \
    _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                             \
      const int ch = k * CPP + chsub;                                                             \
      rb[k] = (rok_ && ch < NCH && ch0 + ch < g.d) ? (pb_ + (size_t)k * CPP * hs2)[b_lane] : 0.f; \
    }                                                                                             \
  } while (0)
#define CCT_WGRAD_STASH()                                                                         \
  do {                                                                                            \
    if (a_ok) {                                                                                   \
      _Pragma("unroll") for (int k = 0; k < NAL; ++k) sa[(arow + 4 * k) * g.ast + ai] = ra[k];    \
    }                                                                                             \
    if (chsub < CPP) {                                                                            \
      _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                           \
        if (k * CPP + chsub < NCH) sb[k * (CPP * PCH) + sb_lane] = rb[k];                         \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  // fragment bases: dout slab row (map) r of block a, half h -> second staged row; patch position of
  // this lane's column (c, kr, kc), half h -> one patch row further down
  int abase[TMB], bbase[TNB];
#pragma unroll
  for (int a = 0; a < TMB; ++a) abase[a] = (a * 32 + r) * g.ast + h * g.ho;
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    const int col = min(n0 + wave * (32 * TNB) + b * 32 + r, g.ncols - 1);
    const int c = col / KK, j = col - c * KK, kr = j / KS, kc = j - kr * KS;
    bbase[b] = (c - ch0) * PCH + (h + kr) * PWS + kc;
  }

  v16f acc[TMB][TNB];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int b = 0; b < TNB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.0f;

  if (s_beg < s_end) CCT_WGRAD_FETCH(s_beg);
  for (int s = s_beg; s < s_end; ++s) {
    CCT_WGRAD_STASH();
    __syncthreads();
    if (s + 1 < s_end) CCT_WGRAD_FETCH(s + 1);
    float fa[2][TMB], fb[2][TNB];
#pragma unroll
    for (int a = 0; a < TMB; ++a) fa[0][a] = sa[abase[a]];
#pragma unroll
    for (int b = 0; b < TNB; ++b) fb[0][b] = sb[bbase[b]];
    // x runs over the output row; two iterations per trip so the fragment buffers alternate statically
    for (int x = 0; x < g.ho; x += 2) {
      const int x1 = min(x + 1, g.ho - 1), x2 = min(x + 2, g.ho - 1);
#pragma unroll
      for (int a = 0; a < TMB; ++a) fa[1][a] = sa[abase[a] + x1];
#pragma unroll
      for (int b = 0; b < TNB; ++b) fb[1][b] = sb[bbase[b] + x1];
#pragma unroll
      for (int a = 0; a < TMB; ++a)
#pragma unroll
        for (int b = 0; b < TNB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0][a], fb[0][b], acc[a][b], 0, 0, 0);
#pragma unroll
      for (int a = 0; a < TMB; ++a) fa[0][a] = sa[abase[a] + x2];
#pragma unroll
      for (int b = 0; b < TNB; ++b) fb[0][b] = sb[bbase[b] + x2];
      if (x + 1 < g.ho) {
#pragma unroll
        for (int a = 0; a < TMB; ++a)
#pragma unroll
          for (int b = 0; b < TNB; ++b)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1][a], fb[1][b], acc[a][b], 0, 0, 0);
      }
    }
    __syncthreads();
  }
#undef CCT_WGRAD_FETCH
#undef CCT_WGRAD_STASH

  float *out = g.out + (size_t)z * g.o * g.ncols;
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    const int col = n0 + wave * (32 * TNB) + b * 32 + r;
    if (col >= g.ncols) continue;
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < g.o) out[(size_t)row * g.ncols + col] = acc[a][b][v];
      }
  }
}

// dst[e] = sum_z ws[z][e], z ascending
__global__ __launch_bounds__(256) void direct_reduce_kernel(float *__restrict__ dst, const float *__restrict__ ws,
                                                            uint32_t n, int splits) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  float s = 0.f;
  for (int z = 0; z < splits; ++z) s += ws[(size_t)z * n + e];
  dst[e] = s;
}

template <int KS, int PW>
static int wgrad_launch(WgradArgs &g, int tmb, int tnb, size_t lds, hipStream_t st) {
  dim3 grid(g.nblocks), block(256);
#define CCT_WGRAD_CASE(TMB, TNB)                                                                       \
  if (tmb == TMB && tnb == TNB) {                                                                      \
    hipLaunchKernelGGL((conv_direct_wgrad_kernel<KS, TMB, TNB, PW>), grid, block, lds, st, g);         \
    CCT_LAUNCH_CHECK();                                                                                \
    return 0;                                                                                          \
  }
  CCT_WGRAD_CASE(2, 1) CCT_WGRAD_CASE(3, 1) CCT_WGRAD_CASE(4, 1)
  CCT_WGRAD_CASE(2, 2) CCT_WGRAD_CASE(3, 2) CCT_WGRAD_CASE(4, 2)
#undef CCT_WGRAD_CASE
  return set_error(CCT_HIP_EINVAL, "conv_direct wgrad: no kernel instance for tile %dx%d", tmb, tnb);
}

static bool wgrad_plan(int batch, int d, int n, int ks, int pad, int o, int *tmb, int *tnb, int *pw,
                       size_t *lds) {
  if (ks != 3 && ks != 5) return false;
  const int ho = n + 2 * pad - ks + 1, hp = ho + ks - 1;
  if (pad < 0 || pad > ks - 1 || ho <= 0 || hp > 32 || batch <= 0 || d <= 0 || o <= 0) return false;
  if ((double)batch * o * ho * ho >= 2147483648.0 || (double)batch * d * n * n >= 2147483648.0 ||
      (double)o * d * ks * ks >= 2147483648.0)
    return false;
  *pw = hp <= 16 ? 16 : 32;
  int best_tmb = 4;
  long best = -1;
  for (int cand = 4; cand >= 2; --cand) {
    const long padded = (long)((o + 32 * cand - 1) / (32 * cand)) * 32 * cand;
    if (best < 0 || padded < best) { best = padded; best_tmb = cand; }
  }
  *tmb = best_tmb;
  // wide column tiles unless they pad the columns noticeably more than narrow ones
  const long ncols = (long)d * ks * ks;
  const long pad2 = (ncols + 255) / 256 * 256, pad1 = (ncols + 127) / 128 * 128;
  *tnb = (pad2 * 100 <= pad1 * 108) ? 2 : 1;
  {
    static const int forced = [] { const char *e = getenv("CCT_HIP_DIRECT_TNB"); return e ? atoi(e) : 0; }();
    if (forced == 1 || forced == 2) *tnb = forced;
  }
  const int ast = (2 * ho) | 1;
  const int nch = (128 * *tnb - 1) / (ks * ks) + 2;
  const int pws = *pw + (((ks - *pw) % 32) + 32) % 32, raw = (ks + 1) * pws;
  const int pch = raw + (((ks * ks - raw) % 32) + 32) % 32;  // WgradStrides<ks, pw>
  *lds = (size_t)(((32 * *tmb * ast + 3) & ~3) + nch * pch) * sizeof(float);
  return *lds <= 64 * 1024;
}

static int conv_direct_wgrad(float *dw, const float *dout, const float *src, int batch, int d, int n, int ks,
                             int pad, int o) {
  int tmb, tnb, pw;
  size_t lds;
  CCT_REQUIRE(wgrad_plan(batch, d, n, ks, pad, o, &tmb, &tnb, &pw, &lds),
              "conv_direct wgrad: geometry not covered (k=%d pad=%d size=%d)", ks, pad, n);
  WgradArgs g;
  g.dout = dout; g.src = src;
  g.batch = batch; g.o = o; g.d = d; g.hs = n; g.pad = pad;
  g.ho = n + 2 * pad - ks + 1;
  g.ncols = d * ks * ks;
  g.chunks = (g.ho + 1) / 2;
  g.ast = (2 * g.ho) | 1;
  g.steps_total = batch * g.chunks;
  g.tiles_m = (uint32_t)((o + 32 * tmb - 1) / (32 * tmb));
  g.tiles_n = (uint32_t)((g.ncols + 128 * tnb - 1) / (128 * tnb));
  g.ntiles = g.tiles_m * g.tiles_n;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  int splits = (int)(2L * cus / g.ntiles);
  if (splits < 1) splits = 1;
  if (splits > g.steps_total) splits = g.steps_total;
  g.steps_per_split = (g.steps_total + splits - 1) / splits;
  splits = (g.steps_total + g.steps_per_split - 1) / g.steps_per_split;
  g.nblocks = g.ntiles * (uint32_t)splits;
  g.div_chunks = make_fastdiv((uint32_t)g.chunks);
  const size_t n_out = (size_t)o * g.ncols;
  if (splits > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)splits * n_out * sizeof(float), &ws);
    if (rc) return rc;
    g.out = (float *)ws;
  } else {
    g.out = dw;
  }
  hipStream_t st = ctx().stream;
  int rc;
  if (ks == 5) rc = pw == 16 ? wgrad_launch<5, 16>(g, tmb, tnb, lds, st) : wgrad_launch<5, 32>(g, tmb, tnb, lds, st);
  else rc = pw == 16 ? wgrad_launch<3, 16>(g, tmb, tnb, lds, st) : wgrad_launch<3, 32>(g, tmb, tnb, lds, st);
  if (rc) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(direct_reduce_kernel, dim3((uint32_t)((n_out + 255) / 256)), dim3(256), 0, st, dw, g.out,
                       (uint32_t)n_out, splits);
    CCT_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_conv_direct_supported(int batch, int depth, int n, int k, int stride, int padding,
                                             int num_outputs) {
  if (stride != 1 || ensure_init() != 0) return 0;
  DirectPlan pl;
  const int m = n + 2 * padding - k + 1;
  // forward: channels = depth, maps = outputs, source n, pad p; data gradient: channels = outputs,
  // maps = depth, source m, pad k-1-p
  int tmb, tnb, pw;
  size_t lds;
  return direct_plan(batch, depth, num_outputs, n, k, padding, &pl) &&
                 direct_plan(batch, num_outputs, depth, m, k, k - 1 - padding, &pl) &&
                 wgrad_plan(batch, depth, n, k, padding, num_outputs, &tmb, &tnb, &pw, &lds)
             ? 1
             : 0;
}

extern "C" size_t cct_hip_conv_direct_slab_floats(int num_outputs, int depth, int k, int for_data_gradient) {
  if (num_outputs <= 0 || depth <= 0 || k <= 0) return 0;
  const int n_c = for_data_gradient ? num_outputs : depth, n_m = for_data_gradient ? depth : num_outputs;
  return (size_t)direct_padded_channels(n_c) * direct_padded_maps(n_m) * k * k;
}

extern "C" int cct_hip_conv_direct_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                                         int for_data_gradient) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(num_outputs > 0 && depth > 0 && k > 0, "conv_direct_slabs: bad dimensions");
  CCT_REQUIRE(slabs != model, "conv_direct_slabs: in-place use");
  const size_t total = cct_hip_conv_direct_slab_floats(num_outputs, depth, k, for_data_gradient);
  CCT_REQUIRE(total < (1ull << 31), "conv_direct_slabs: model too large");
  // forward slabs: [depth][outputs][k*k]; data-gradient slabs: [outputs][depth][k*k] reversed
  const int n_c = for_data_gradient ? num_outputs : depth, n_m = for_data_gradient ? depth : num_outputs;
  const int p_m = direct_padded_maps(n_m);
  hipLaunchKernelGGL(direct_slab_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx().stream,
                     slabs, model, n_c, n_m, p_m, (uint32_t)total, k * k, for_data_gradient ? 1 : 0,
                     make_fastdiv((uint32_t)(k * k)), make_fastdiv((uint32_t)p_m));
  CCT_LAUNCH_CHECK();
  return 0;
}

extern "C" int cct_hip_conv_direct_forward(float *output, const float *input, const float *slabs,
                                           const float *bias, int batch, int depth, int n, int k, int padding,
                                           int num_outputs) {
  CCT_ENSURE_INIT();
  if (batch <= 0) return 0;
  return conv_direct(slabs, input, output, bias, batch, depth, num_outputs, n, k, padding);
}

extern "C" int cct_hip_conv_direct_backward_data(float *input_grad, const float *output_grad,
                                                 const float *slabs, int batch, int depth, int n, int k,
                                                 int padding, int num_outputs) {
  CCT_ENSURE_INIT();
  if (batch <= 0) return 0;
  const int m = n + 2 * padding - k + 1;
  return conv_direct(slabs, output_grad, input_grad, nullptr, batch, num_outputs, depth, m, k,
                     k - 1 - padding);
}

extern "C" int cct_hip_conv_direct_backward_weights(float *model_grad, const float *output_grad,
                                                    const float *input, int batch, int depth, int n, int k,
                                                    int padding, int num_outputs) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(batch > 0, "conv_direct_backward_weights: empty batch");
  return conv_direct_wgrad(model_grad, output_grad, input, batch, depth, n, k, padding, num_outputs);
}
