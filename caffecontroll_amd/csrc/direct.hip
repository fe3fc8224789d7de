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
// pixels (pixels are numbered across the whole batch, so a tile may straddle images; an image whose
// padded rows exceed a patch row is cut into column bands that are numbered like images, see
// DirectArgs::wv).  KS is 3, 5 or 7.  The contraction index is consumed two*CP channels per step:
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
#include <type_traits>

#include "cct_common.h"
#include "mfma_common.h"

namespace cct {

struct DirectArgs {
  const float *wt;    // slab buffer [kc padded to 4][mtot padded to whole tiles][KS*KS], zero padding
  const float *src;   // [batch][kc][hs][hs]
  float *dst;         // [batch][mtot][ho][ho]
  const float *bias;  // [mtot] or null
  int relu;           // epilogue clamps at zero (ReLU of the layer that follows, folded in)
  const float *mask;  // same shape as dst, or null: store 0 where mask <= 0 (data gradient through the ReLU before the layer)
  int batch, kc, mtot, hs, ho, pad;
  int hp;             // ho + KS - 1 = hs + 2*pad: rows (and columns) of a zero-padded source image
  int pr;             // patch rows per channel
  int nsteps;         // ceil(kc / channels per step)
  int slab_stride;    // floats between channels of the slab buffer (padded map count * KS*KS)
  uint32_t src_img_stride, dst_img_stride;  // floats between images (>= kc*hs*hs, mtot*ho*ho: channel-slice views)
  uint32_t ptot;      // batch * ho * ho
  uint32_t tiles_m, ntiles;
  FastDiv div_ho, div_ho2, div_hp, div_pr;
  int cs;             // 16-row kernel: floats between the channels of a patch (pr * PW + 16)
  FastDiv div_cs;
  // 16-row kernel, data gradient of a strided layer: the output maps are (channel, row phase, column
  // phase) triples of the layer's input gradient, pixel (I, J) of map (c, pi, pj) is stored at
  // dst[img][c][S*I + pi - spad][S*J + pj - spad] of a [batch][sd][shs][shs] tensor (ss = S; 0 = plain output)
  int ss, shs, spad, sd;
  // channel groups of a grouped convolution, all in this launch: group q reads channels q*kc .. of src and
  // writes maps q*mtot .. of dst with the slab buffer at wt + q*wt_group_floats; tile ids run group by group
  int groups;
  uint32_t tiles_per_group, wt_group_floats;
  // 32-row kernel, images wider than a patch row: every image is cut into `nbands` column bands of `wv` output
  // columns (the last one may reach past the right edge), and a band is numbered like an image of its own --
  // tile pixel p = ((img * nbands + band) * ho + y) * wv + x -- so a tile's patch holds wv + KS - 1 columns of
  // the source rows it touches instead of whole rows.  One band of wv = ho columns otherwise.
  int wv, nbands;
  uint32_t vpix;      // wv * ho: pixels of a band
  FastDiv div_wv, div_vpix, div_nbands;
};

constexpr int kDirect16PatchLoads = 11;  // the 16-row kernel stages four channels per step

// source elements per lane per step, at most
constexpr int kDirectPatchLoads = 8;

// Fragments of contraction index idx = cp*KS*KS + j (idx is a constant after unrolling): weights of
// tap j of channel pair cp for TMB row blocks, source elements under tap j for TNB pixel blocks.
// wa[cp][a] / pb[cp][b]: LDS word of this lane's first weight of row block a / first source element of pixel
// block b, for channel pair cp, within the stage being read.
template <int KS, int TMB, int TNB, int CP, int PW>
__device__ __forceinline__ void direct_frags(float (&fa)[TMB], float (&fb)[TNB], const float *__restrict__ sm,
                                             const int (&wa)[CP][TMB], const int (&pb)[CP][TNB], int idx) {
  constexpr int KK = KS * KS;
  const int cp = idx / KK, j = idx % KK, u = j / KS, v = j % KS;
#pragma unroll
  for (int a = 0; a < TMB; ++a) fa[a] = sm[wa[cp][a] + j];
#pragma unroll
  for (int b = 0; b < TNB; ++b) fb[b] = sm[pb[cp][b] + u * PW + v];
}

// Wavefronts per SIMD the register allocation must leave room for, by accumulator blocks of the tile: the
// workgroups resident on a compute unit are what hides the barrier of every step (and the tail of the grid),
// so a tile must not lose a resident workgroup to a handful of address registers.
constexpr int direct_waves_per_simd(int blocks) {
  return blocks <= 1 ? 8 : blocks == 2 ? 7 : blocks == 3 ? 5 : blocks == 4 ? 4 : blocks <= 6 ? 3 : 2;
}

template <int KS, int TMB, int TNB, int CP, int PW>
__global__ __launch_bounds__(256, direct_waves_per_simd(TMB * TNB)) void conv_direct_kernel(const DirectArgs g) {
  constexpr int KK = KS * KS, BM = 32 * TMB, BN = 128 * TNB, NC = 2 * CP;
  constexpr int ASZ = NC * BM * KK;           // floats of weight slabs per stage
  constexpr int ASZP = (ASZ + 255) / 256 * 256;  // LDS room for them: whole 64-lane 16-byte loads
  constexpr int SLAB4 = BM * KK / 4;          // 16-byte vectors per slab
  constexpr int NA4 = (ASZP / 4 + 255) / 256;  // 16-byte vectors per lane per stage
  constexpr int NPL = kDirectPatchLoads;
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // known to be wave-uniform
  const int r = lane & 31, h = lane >> 5;
  const int psz = (NC * g.pr * PW + 63) & ~63;  // floats of patches per stage: whole 64-lane loads
  const int stage = ASZP + psz;

  uint32_t id = xcd_remap(blockIdx.x, g.ntiles);
  const uint32_t grp = g.groups > 1 ? id / g.tiles_per_group : 0u;  // workgroup-uniform
  id -= grp * g.tiles_per_group;
  const uint32_t tn = id / g.tiles_m, tm = id - tn * g.tiles_m;
  const int m0 = tm * BM;
  const uint32_t p0 = tn * BN;
  const int ho2 = g.ho * g.ho;

  // first patch row: the virtual row of the tile's first pixel (bands stacked like images, hp rows each)
  const uint32_t img0 = fdiv(p0, g.div_vpix);
  const uint32_t y0 = fdiv(p0 - img0 * g.vpix, g.div_wv);
  const int v_lo = img0 * g.hp + y0;

  // ---- per-lane loader state -------------------------------------------------------------
  // Operands go from global memory straight into LDS (global_load_lds): a wave's load writes its
  // 64 lanes' data to consecutive LDS addresses, so LDS element e is fetched by lane e % 64 of the
  // wave-instruction that covers e.  Every address is a wave-uniform base that advances per step
  // plus a per-lane offset fixed for the whole tile.
  //   weights: the slab buffer is padded with zero rows and zero channels up to whole tiles and
  //            whole steps, so the loads need no bounds tests;
  //   source : patch element e = (channel c, patch row, patch column); elements outside the image
  //            get the out-of-range offset and arrive as zeros, so do channels past the last one
  //            in the final step.
  uint32_t aoff[NA4];
#pragma unroll
  for (int i = 0; i < NA4; ++i) {
    const int e4 = tid + i * 256;
    const int c = e4 / SLAB4, f = (e4 - c * SLAB4) * 4;
    // bytes; the lanes past the slabs' end fill the padding of the LDS region with zeros
    aoff[i] = e4 < ASZ / 4 ? (uint32_t)(c * g.slab_stride + f) * 4u : kOutOfRange;
  }
  // byte offsets; in the final step the lanes of channels past the last one fetch nothing (that test is redone
  // where it is needed, in the final step's loads, rather than kept in a second set of registers)
  uint32_t psrc[NPL];
  const int last_channels = g.kc - (g.nsteps - 1) * NC;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const uint32_t e = tid + i * 256;
    const uint32_t pc = e % PW, rest = e / PW;
    const uint32_t c = fdiv(rest, g.div_pr), prow = rest - c * g.pr;
    const uint32_t v = v_lo + prow;
    const uint32_t vi = fdiv(v, g.div_hp), img = fdiv(vi, g.div_nbands), band = vi - img * g.nbands;
    const int srow = (int)(v - vi * g.hp) - g.pad, scol = (int)(band * g.wv + pc) - g.pad;
    const bool ok = c < (uint32_t)NC && img < (uint32_t)g.batch && pc < (uint32_t)(g.wv + KS - 1) &&
                    (unsigned)srow < (unsigned)g.hs && (unsigned)scol < (unsigned)g.hs;
    psrc[i] = ok ? (img * g.src_img_stride + (c * g.hs + srow) * g.hs + scol) * 4u : kOutOfRange;
  }
  const uint32_t a_step = (uint32_t)NC * g.slab_stride * 4u, b_step = (uint32_t)NC * g.hs * g.hs * 4u;  // bytes
  const rsrc_t a_rsrc = make_rsrc(g.wt + (size_t)grp * g.wt_group_floats + (size_t)m0 * KK),
               b_rsrc = make_rsrc(g.src + (size_t)grp * g.kc * g.hs * g.hs);
  const int wave_elem0 = wave * 64;  // first element of this wave within a 256-element pass

// global -> LDS stage s for step t (asynchronous; completion = vmcnt)
#define CCT_DIRECT_ISSUE(t, s)                                                                 \
  do {                                                                                         \
    float *st_ = smem + (s) * stage;                                                           \
    const uint32_t ga_ = (uint32_t)(t) * a_step, gb_ = (uint32_t)(t) * b_step;                 \
    _Pragma("unroll") for (int i = 0; i < NA4; ++i) {                                          \
      if (i * 256 + wave_elem0 < ASZP / 4)                                                     \
        lds_dma16(a_rsrc, aoff[i], ga_, st_ + (i * 256 + wave_elem0) * 4);                     \
    }                                                                                          \
    const bool last_ = (t) == g.nsteps - 1;                                                    \
    _Pragma("unroll") for (int i = 0; i < NPL; ++i) {                                          \
      if (i * 256 + wave_elem0 < psz)                                                          \
        lds_dma4(b_rsrc,                                                                       \
                 (last_ && (int)fdiv((uint32_t)(tid + i * 256) / PW, g.div_pr) >= last_channels) ? kOutOfRange \
                                                                                                : psrc[i], \
                 gb_, st_ + ASZP + i * 256 + wave_elem0);                                      \
    }                                                                                          \
  } while (0)

  // ---- per-lane fragment bases --------------------------------------------------------------
  const int abase = h * (BM * KK) + r * KK;
  int bbase[TNB];
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    uint32_t p = p0 + wave * (32 * TNB) + b * 32 + r;
    p = min(p, g.ptot - 1);
    const uint32_t vi = fdiv(p, g.div_vpix);
    const uint32_t pix = p - vi * g.vpix;
    const uint32_t y = fdiv(pix, g.div_wv), x = pix - y * g.wv;
    bbase[b] = ASZP + h * (g.pr * PW) + (int)(vi * g.hp + y - v_lo) * PW + (int)x;
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

  // Fragment addresses of both stages as registers of their own (seen as one base plus constants, they would be
  // re-added before every read: the paired LDS read reaches 255 words beyond its address register).  Vector ALU
  // instructions and MFMAs of one SIMD do not overlap, so address arithmetic in the loop is MFMA time lost.
  int wa2[2][CP][TMB], pb2[2][CP][TNB];
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
    for (int cp = 0; cp < CP; ++cp) {
#pragma unroll
      for (int a = 0; a < TMB; ++a) {
        wa2[s2][cp][a] = s2 * stage + abase + cp * (2 * BM * KK) + a * (32 * KK);
        asm volatile("" : "+v"(wa2[s2][cp][a]));
      }
#pragma unroll
      for (int b = 0; b < TNB; ++b) {
        pb2[s2][cp][b] = s2 * stage + bbase[b] + cp * pair_stride;
        asm volatile("" : "+v"(pb2[s2][cp][b]));
      }
    }

  // One step.  FAST: the stage read is the compile-time constant P and the step fetched, t + 1, exists and is not
  // the final one (its loads need no choice between the two offset sets); else the stage is t & 1 and the loads
  // are chosen at run time.  The loop runs FAST steps in pairs and leaves the last two or three to the other form.
  auto step = [&](auto fast_c, auto stage_c, int t) {
    constexpr bool FAST = decltype(fast_c)::value;
    constexpr int P = decltype(stage_c)::value;
    // every wave finished reading the other stage before the barrier that ended step t-1
    if constexpr (FAST) {
      float *st_ = smem + (P ^ 1) * stage;
      const uint32_t ga_ = (uint32_t)(t + 1) * a_step, gb_ = (uint32_t)(t + 1) * b_step;
      // loads this wavefront makes per step (counts as scalar registers read afresh every step: a loop-invariant
      // "does load i exist" flag would be kept as a lane mask and turned back into a branch with vector
      // instructions)
      int na_ = (ASZP / 4 - wave_elem0 + 255) / 256, np_ = (psz - wave_elem0 + 255) / 256;
      asm volatile("" : "+s"(na_), "+s"(np_));
#pragma unroll
      for (int i = 0; i < NA4; ++i) {
        if (__builtin_expect(i < na_, 1)) lds_dma16(a_rsrc, aoff[i], ga_, st_ + (i * 256 + wave_elem0) * 4);
      }
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        if (__builtin_expect(i < np_, 1)) lds_dma4(b_rsrc, psrc[i], gb_, st_ + ASZP + i * 256 + wave_elem0);
      }
    } else {
      if (t + 1 < g.nsteps) CCT_DIRECT_ISSUE(t + 1, (t & 1) ^ 1);
    }
    const float *sm = smem;
    int wa[CP][TMB], pb[CP][TNB];
#pragma unroll
    for (int cp = 0; cp < CP; ++cp) {
#pragma unroll
      for (int a = 0; a < TMB; ++a)
        wa[cp][a] = FAST ? wa2[P][cp][a] : (t & 1) * stage + abase + cp * (2 * BM * KK) + a * (32 * KK);
#pragma unroll
      for (int b = 0; b < TNB; ++b) pb[cp][b] = FAST ? pb2[P][cp][b] : (t & 1) * stage + bbase[b] + cp * pair_stride;
    }
    // Contraction indices are taken two at a time (neighbouring taps sit in neighbouring LDS words,
    // which lets the compiler fetch both with one ds_read2); the fragments of pair q+1 are
    // requested before the MFMAs of pair q.
    constexpr int NI = CP * KK, NQ = (NI + 1) / 2;
    float fa[2][2][TMB], fb[2][2][TNB];
    direct_frags<KS, TMB, TNB, CP, PW>(fa[0][0], fb[0][0], sm, wa, pb, 0);
    if (NI > 1) direct_frags<KS, TMB, TNB, CP, PW>(fa[0][1], fb[0][1], sm, wa, pb, 1);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int nb = (q + 1) & 1, cb = q & 1;
      if (2 * q + 2 < NI) direct_frags<KS, TMB, TNB, CP, PW>(fa[nb][0], fb[nb][0], sm, wa, pb, 2 * q + 2);
      if (2 * q + 3 < NI) direct_frags<KS, TMB, TNB, CP, PW>(fa[nb][1], fb[nb][1], sm, wa, pb, 2 * q + 3);
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
  };
  {
    int t = 0;
    for (; t + 3 < g.nsteps; t += 2) {
      step(std::true_type{}, std::integral_constant<int, 0>{}, t);
      step(std::true_type{}, std::integral_constant<int, 1>{}, t + 1);
    }
    for (; t < g.nsteps; ++t) step(std::false_type{}, std::integral_constant<int, 0>{}, t);
  }
#undef CCT_DIRECT_ISSUE

  // ---- epilogue: accumulator register v of lane (r,h) is row 8*(v/4) + 4*h + v%4, column r ----
#pragma unroll
  for (int b = 0; b < TNB; ++b) {
    const uint32_t p = p0 + wave * (32 * TNB) + b * 32 + r;
    if (p >= g.ptot) continue;
    const uint32_t vi = fdiv(p, g.div_vpix), img = fdiv(vi, g.div_nbands), band = vi - img * g.nbands;
    const uint32_t bpix = p - vi * g.vpix, by = fdiv(bpix, g.div_wv), xr = band * g.wv + (bpix - by * g.wv);
    if (xr >= (uint32_t)g.ho) continue;  // the last band's columns past the right edge
    const size_t pix = (size_t)img * g.dst_img_stride + (size_t)grp * g.mtot * ho2 + (by * g.ho + xr);
    float *out = g.dst + pix;
    const float *gbias = g.bias ? g.bias + (size_t)grp * g.mtot : nullptr;
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < g.mtot) {
          float y = acc[a][b][v] + (gbias ? gbias[row] : 0.f);
          if (g.mask && !(g.mask[pix + (size_t)row * ho2] > 0.f)) y = 0.f;
          out[(size_t)row * ho2] = (g.relu && !(y > 0.f)) ? 0.f : y;
        }
      }
  }
}

// The same convolution on 16-row MFMA tiles (v_mfma_f32_16x16x4_f32: 16 maps x 16 pixels, four
// contraction indices) for map counts that 32-row blocks would pad by half a block: 48 maps (one
// group of CaffeNet conv2's data gradient) run as three 16-row blocks instead of two 32-row blocks
// of which a quarter is zeros.  Same slab buffer, same patch layout, same two-stage pipeline; what
// changes is the fragment geometry: a step takes FOUR channels, lanes 16q..16q+15 hold channel q of
// the step for map (or pixel) lane % 16, and accumulator register v of lane (r, q) is row 4*q + v,
// column r of its 16 x 16 block.  One tile covers all maps (BM = 16*TM16) x 128*TNB pixels; a
// wavefront owns 2*TNB blocks of 16 consecutive pixels.
typedef float v4f __attribute__((ext_vector_type(4)));

// wavefronts per SIMD the register allocation must leave room for, by accumulator registers of the tile (what the
// instances held before their fragment addresses became registers)
constexpr int direct16_waves_per_simd(int acc_regs) {
  return acc_regs <= 8 ? 8 : acc_regs <= 16 ? 6 : acc_regs <= 24 ? 5 : acc_regs <= 48 ? 4 : acc_regs <= 80 ? 3 : 2;
}

// wa[a] / pb[b]: LDS word of this lane's first weight of row block a / first source element of pixel block b within
// the stage being read.
template <int KS, int TM16, int NB, int PW>
__device__ __forceinline__ void direct16_frags(float (&fa)[TM16], float (&fb)[NB], const float *__restrict__ sm,
                                               const int (&wa)[TM16], const int (&pb)[NB], int j) {
  const int u = j / KS, v = j % KS;
#pragma unroll
  for (int a = 0; a < TM16; ++a) fa[a] = sm[wa[a] + j];
#pragma unroll
  for (int b = 0; b < NB; ++b) fb[b] = sm[pb[b] + u * PW + v];
}

template <int KS, int TM16, int TNB, int PW>
__global__ __launch_bounds__(256, direct16_waves_per_simd(TM16 * 2 * TNB * 4)) void conv_direct16_kernel(
    const DirectArgs g) {
  constexpr int KK = KS * KS, BM = 16 * TM16, BN = 128 * TNB, NC = 4, NB = 2 * TNB;
  constexpr int ASZ = NC * BM * KK;
  constexpr int ASZP = (ASZ + 255) / 256 * 256;
  constexpr int SLAB4 = BM * KK / 4;
  constexpr int NA4 = (ASZP / 4 + 255) / 256;
  constexpr int NPL = kDirect16PatchLoads;
  static_assert(BM * KK % 4 == 0, "weight slabs are copied in 16-byte vectors");
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  // channels of a patch lie pr*PW + 16 floats apart: the four channel groups of a fragment read
  // then fall on two bank halves instead of one
  const int psz = (NC * g.cs + 63) & ~63;
  const int stage = ASZP + psz;

  uint32_t tn = xcd_remap(blockIdx.x, g.ntiles);  // one map tile: the tile id is (group, pixel tile)
  const uint32_t grp = g.groups > 1 ? tn / g.tiles_per_group : 0u;  // workgroup-uniform
  tn -= grp * g.tiles_per_group;
  const uint32_t p0 = tn * BN;
  const int ho2 = g.ho * g.ho;
  const uint32_t img0 = fdiv(p0, g.div_ho2);
  const uint32_t y0 = fdiv(p0 - img0 * ho2, g.div_ho);
  const int v_lo = img0 * g.hp + y0;

  uint32_t aoff[NA4];
#pragma unroll
  for (int i = 0; i < NA4; ++i) {
    const int e4 = tid + i * 256;
    const int c = e4 / SLAB4, f = (e4 - c * SLAB4) * 4;
    // bytes; the lanes past the slabs' end fill the padding of the LDS region with zeros
    aoff[i] = e4 < ASZ / 4 ? (uint32_t)(c * g.slab_stride + f) * 4u : kOutOfRange;
  }
  // byte offsets; in the final step the lanes of channels past the last one fetch nothing (tested where it is
  // needed, in the final step's loads)
  uint32_t psrc[NPL];
  const int last_channels = g.kc - (g.nsteps - 1) * NC;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const uint32_t e = tid + i * 256;
    const uint32_t c = fdiv(e, g.div_cs), rem = e - c * g.cs;
    const uint32_t prow = rem / PW, pc = rem % PW;
    const uint32_t v = v_lo + prow;
    const uint32_t img = fdiv(v, g.div_hp);
    const int srow = (int)(v - img * g.hp) - g.pad, scol = (int)pc - g.pad;
    const bool ok = c < (uint32_t)NC && prow < (uint32_t)g.pr && img < (uint32_t)g.batch && (unsigned)srow < (unsigned)g.hs &&
                    (unsigned)scol < (unsigned)g.hs;
    psrc[i] = ok ? (img * g.src_img_stride + (c * g.hs + srow) * g.hs + scol) * 4u : kOutOfRange;
  }
  const uint32_t a_step = (uint32_t)NC * g.slab_stride * 4u, b_step = (uint32_t)NC * g.hs * g.hs * 4u;
  const rsrc_t a_rsrc = make_rsrc(g.wt + (size_t)grp * g.wt_group_floats),
               b_rsrc = make_rsrc(g.src + (size_t)grp * g.kc * g.hs * g.hs);
  const int wave_elem0 = wave * 64;

#define CCT_DIRECT16_ISSUE(t, s)                                                               \
  do {                                                                                         \
    float *st_ = smem + (s) * stage;                                                           \
    const uint32_t ga_ = (uint32_t)(t) * a_step, gb_ = (uint32_t)(t) * b_step;                 \
    _Pragma("unroll") for (int i = 0; i < NA4; ++i) {                                          \
      if (i * 256 + wave_elem0 < ASZP / 4)                                                     \
        lds_dma16(a_rsrc, aoff[i], ga_, st_ + (i * 256 + wave_elem0) * 4);                     \
    }                                                                                          \
    const bool last_ = (t) == g.nsteps - 1;                                                    \
    _Pragma("unroll") for (int i = 0; i < NPL; ++i) {                                          \
      if (i * 256 + wave_elem0 < psz)                                                          \
        lds_dma4(b_rsrc,                                                                       \
                 (last_ && (int)fdiv((uint32_t)(tid + i * 256), g.div_cs) >= last_channels) ? kOutOfRange : psrc[i], \
                 gb_, st_ + ASZP + i * 256 + wave_elem0);                                      \
    }                                                                                          \
  } while (0)

  const int abase = q * (BM * KK) + r * KK;
  int bbase[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    uint32_t p = p0 + wave * (32 * TNB) + b * 16 + r;
    p = min(p, g.ptot - 1);
    const uint32_t img = fdiv(p, g.div_ho2);
    const uint32_t pix = p - img * ho2;
    const uint32_t y = fdiv(pix, g.div_ho), x = pix - y * g.ho;
    bbase[b] = ASZP + q * g.cs + (int)(img * g.hp + y - v_lo) * PW + (int)x;
  }

  v4f acc[TM16][NB];
#pragma unroll
  for (int a = 0; a < TM16; ++a)
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[a][b][e] = 0.0f;

  CCT_DIRECT16_ISSUE(0, 0);
  lds_dma_wait();
  __syncthreads();

  // Fragment addresses of both stages as registers of their own, the step loop in pairs with the stage a
  // compile-time constant, scalar load counts: as in conv_direct_kernel, no vector ALU instruction is left in the loop.
  int wa2[2][TM16], pb2[2][NB];
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
    for (int a = 0; a < TM16; ++a) {
      wa2[s2][a] = s2 * stage + abase + a * (16 * KK);
      asm volatile("" : "+v"(wa2[s2][a]));
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      pb2[s2][b] = s2 * stage + bbase[b];
      asm volatile("" : "+v"(pb2[s2][b]));
    }
  }

  auto step = [&](auto fast_c, auto stage_c, int t) {
    constexpr bool FAST = decltype(fast_c)::value;
    constexpr int P = decltype(stage_c)::value;
    if constexpr (FAST) {
      float *st_ = smem + (P ^ 1) * stage;
      const uint32_t ga_ = (uint32_t)(t + 1) * a_step, gb_ = (uint32_t)(t + 1) * b_step;
      int na_ = (ASZP / 4 - wave_elem0 + 255) / 256, np_ = (psz - wave_elem0 + 255) / 256;
      asm volatile("" : "+s"(na_), "+s"(np_));
#pragma unroll
      for (int i = 0; i < NA4; ++i) {
        if (__builtin_expect(i < na_, 1)) lds_dma16(a_rsrc, aoff[i], ga_, st_ + (i * 256 + wave_elem0) * 4);
      }
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        if (__builtin_expect(i < np_, 1)) lds_dma4(b_rsrc, psrc[i], gb_, st_ + ASZP + i * 256 + wave_elem0);
      }
    } else {
      if (t + 1 < g.nsteps) CCT_DIRECT16_ISSUE(t + 1, (t & 1) ^ 1);
    }
    const float *sm = smem;
    int wa[TM16], pb[NB];
#pragma unroll
    for (int a = 0; a < TM16; ++a) wa[a] = FAST ? wa2[P][a] : (t & 1) * stage + abase + a * (16 * KK);
#pragma unroll
    for (int b = 0; b < NB; ++b) pb[b] = FAST ? pb2[P][b] : (t & 1) * stage + bbase[b];
    // taps two at a time (neighbouring taps sit in neighbouring LDS words); the fragments of pair
    // n+1 are requested before the MFMAs of pair n
    constexpr int NI = KK, NQ = (NI + 1) / 2;
    float fa[2][2][TM16], fb[2][2][NB];
    direct16_frags<KS, TM16, NB, PW>(fa[0][0], fb[0][0], sm, wa, pb, 0);
    direct16_frags<KS, TM16, NB, PW>(fa[0][1], fb[0][1], sm, wa, pb, 1);
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
      const int nb = (n + 1) & 1, cb = n & 1;
      if (2 * n + 2 < NI) direct16_frags<KS, TM16, NB, PW>(fa[nb][0], fb[nb][0], sm, wa, pb, 2 * n + 2);
      if (2 * n + 3 < NI) direct16_frags<KS, TM16, NB, PW>(fa[nb][1], fb[nb][1], sm, wa, pb, 2 * n + 3);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (2 * n + e < NI) {
#pragma unroll
          for (int a2 = 0; a2 < TM16; ++a2)
#pragma unroll
            for (int b2 = 0; b2 < NB; ++b2)
              acc[a2][b2] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[cb][e][a2], fb[cb][e][b2], acc[a2][b2], 0, 0, 0);
        }
      }
      {
        constexpr int NR = TM16 + NB, NM = 2 * TM16 * NB, PER = NM / (NR + 1) > 0 ? NM / (NR + 1) : 1;
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
  };
  {
    int t = 0;
    for (; t + 3 < g.nsteps; t += 2) {
      step(std::true_type{}, std::integral_constant<int, 0>{}, t);
      step(std::true_type{}, std::integral_constant<int, 1>{}, t + 1);
    }
    for (; t < g.nsteps; ++t) step(std::false_type{}, std::integral_constant<int, 0>{}, t);
  }
#undef CCT_DIRECT16_ISSUE

  // ---- epilogue: accumulator register v of lane (r, q) is row 4*q + v, column r ----
  if (g.ss) {
    // maps are (channel, row phase, column phase) of a strided layer's input gradient
    const int S = g.ss, S2 = S * S, shs2 = g.shs * g.shs;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const uint32_t p = p0 + wave * (32 * TNB) + b * 16 + r;
      if (p >= g.ptot) continue;
      const uint32_t img = fdiv(p, g.div_ho2);
      const uint32_t pix = p - img * ho2;
      const int I = (int)fdiv(pix, g.div_ho), J = (int)pix - I * g.ho;
      float *out = g.dst + (size_t)img * g.sd * shs2;
#pragma unroll
      for (int a = 0; a < TM16; ++a) {
        const int row0 = a * 16 + 4 * q;  // this lane's four rows: row0 .. row0 + 3
        if (S == 4) {
          // rows 4*q .. 4*q+3 of block a are the four column phases of (channel a, row phase q): four
          // consecutive floats of one image row
          const int i = 4 * I + q - g.spad, j0 = 4 * J - g.spad;
          if (a >= g.sd || (unsigned)i >= (unsigned)g.shs) continue;
          float *o = out + ((size_t)a * g.shs + i) * g.shs + j0;
          if (j0 >= 0 && j0 + 3 < g.shs) {
            *reinterpret_cast<v4f *>(o) = acc[a][b];
          } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
              if ((unsigned)(j0 + v) < (unsigned)g.shs) o[v] = acc[a][b][v];
          }
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int row = row0 + v;
            if (row >= g.mtot) continue;
            const int c = row / S2, rem = row - c * S2, pi = rem / S, pj = rem - pi * S;
            const int i = S * I + pi - g.spad, j = S * J + pj - g.spad;
            if ((unsigned)i < (unsigned)g.shs && (unsigned)j < (unsigned)g.shs)
              out[((size_t)c * g.shs + i) * g.shs + j] = acc[a][b][v];
          }
        }
      }
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const uint32_t p = p0 + wave * (32 * TNB) + b * 16 + r;
    if (p >= g.ptot) continue;
    const uint32_t img = fdiv(p, g.div_ho2);
    const size_t pix = (size_t)img * g.dst_img_stride + (size_t)grp * g.mtot * ho2 + (p - img * ho2);
    float *out = g.dst + pix;
    const float *gbias = g.bias ? g.bias + (size_t)grp * g.mtot : nullptr;
#pragma unroll
    for (int a = 0; a < TM16; ++a)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int row = a * 16 + 4 * q + v;
        if (row < g.mtot) {
          float y = acc[a][b][v] + (gbias ? gbias[row] : 0.f);
          if (g.mask && !(g.mask[pix + (size_t)row * ho2] > 0.f)) y = 0.f;
          out[(size_t)row * ho2] = (g.relu && !(y > 0.f)) ? 0.f : y;
        }
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
  // blockIdx.y = channel group: its own [n_m or n_c][..][kk] block of the model, its own slab buffer
  wt += (size_t)blockIdx.y * total;
  w += (size_t)blockIdx.y * n_c * n_m * kk;
  const uint32_t cm = fdiv(e, div_kk), j = e - cm * kk;
  const uint32_t c = fdiv(cm, div_m), m = cm - c * p_m;
  float v = 0.f;
  if (c < (uint32_t)n_c && m < (uint32_t)n_m)
    v = reversed ? w[((size_t)c * n_m + m) * kk + (kk - 1 - j)] : w[((size_t)m * n_c + c) * kk + j];
  wt[e] = v;
}

struct DirectPlan {
  int ks, tmb, tnb, cp, pw, pr;
  int wv, nbands;  // column bands of a wide image (DirectArgs); wv = output width and one band otherwise
  int tm16;  // > 0: the 16-row kernel with this many row blocks (one map tile); tmb is unused then
  size_t lds;
};

// 16-row blocks of a map count that 32-row blocks would pad by half a block, if the 16-row kernel has
// an instance for it (1, 3 or 5 blocks in a single tile), else 0.
static int direct_tm16(int mtot) {
  const int blocks16 = (mtot + 15) / 16;
  return (blocks16 & 1) && blocks16 <= 5 ? blocks16 : 0;
}

// Chooses the kernel instance for a geometry; returns false when the direct path does not cover it.
static bool direct_plan(int batch, int kc, int mtot, int hs, int ks, int pad, DirectPlan *pl, int groups = 1) {
  if (ks != 3 && ks != 5 && ks != 7) return false;
  if (pad < 0 || pad > ks - 1 || batch <= 0 || kc <= 0 || mtot <= 0 || groups <= 0) return false;
  const int ho = hs + 2 * pad - ks + 1, hp = ho + ks - 1;
  if (ho <= 0) return false;
  // Patch rows hold 16, 32 or 64 floats.  A wider padded image is cut into column bands (32-row kernel only),
  // each numbered like an image of `wv` columns: the fewest bands that fit 64-float rows, or 32-float rows (more
  // patch rows per load, which is what lets a tile of narrow bands fit); the tile estimate below chooses.  An
  // image of 33..64 padded columns whose rows are too many for one patch (7 x 7 filters) falls back to bands of
  // 32-float rows as well.
  struct Bands { int nbands, wv, pw; } layouts[2];
  int nlayouts = 0;
  if (hp <= 64) {
    layouts[nlayouts++] = {1, ho, hp <= 16 ? 16 : hp <= 32 ? 32 : 64};
    if (hp > 32) {
      const int widest = 32 - (ks - 1), nb = (ho + widest - 1) / widest;
      layouts[nlayouts++] = {nb, (ho + nb - 1) / nb, 32};
    }
  } else {
    for (int row = 64; row >= 32; row /= 2) {
      const int widest = row - (ks - 1), nb = (ho + widest - 1) / widest;
      layouts[nlayouts++] = {nb, (ho + nb - 1) / nb, row};
    }
  }
  // buffer loads address a tensor through 32-bit byte offsets
  if ((double)batch * kc * groups * hs * hs >= 536870912.0) return false;
  const int cp = ks == 3 ? 2 : 1;
  pl->wv = ho; pl->nbands = 1;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  const int padded = direct_padded_maps(mtot);
  // tuning override "<map blocks><pixel blocks>", e.g. 22; 161 / 162 = the 16-row kernel with 128 / 256 pixels
  const int forced = tuning().direct_tile;
  pl->tm16 = 0;
  if (const int tm16 = direct_tm16(mtot); tm16 && ks <= 5 && hp <= 64 && (forced == 0 || forced == 161 || forced == 162)) {
    const int pw = layouts[0].pw;
    const long ptot = (long)batch * ho * ho;
    if (ptot >= 2147483648L) return false;
    // 256-pixel tiles (seven LDS reads per twelve MFMAs of a tap instead of five per six) where the launch still
    // has some four of them per compute unit -- measured 1.5-3 % faster on the data gradients of CaffeNet's conv1
    // (sixteen phases) and grouped conv2 -- else 128-pixel tiles
    const bool wide_first = forced == 162 || (forced == 0 && (long)groups * ((ptot + 255) / 256) >= 4L * cus);
    for (int trial = 0; trial < 2; ++trial) {
      const int tnb = (trial == 0) == wide_first ? 2 : 1;
      if ((forced == 161 && tnb == 2) || (forced == 162 && tnb == 1)) continue;
      const int bn = 128 * tnb;
      const int rows = (ho - 1 + bn - 1) / ho + 1, imgs = (ho * ho - 1 + bn - 1) / (ho * ho) + 1;
      const int pr = rows - 1 + (imgs - 1) * (ks - 1) + ks;
      const long patch = 4L * (pr * pw + 16);
      const size_t lds =
          2 * (size_t)((4 * 16 * tm16 * ks * ks + 255) / 256 * 256 + (patch + 63) / 64 * 64) * sizeof(float);
      if (patch > 256L * kDirect16PatchLoads || lds > 64 * 1024) continue;
      pl->ks = ks; pl->tmb = 0; pl->tnb = tnb; pl->cp = 2; pl->pw = pw; pl->pr = pr; pl->tm16 = tm16; pl->lds = lds;
      return true;
    }
  }
  // Candidate tiles: map tiles that divide the padded map count (the slab layout does not depend
  // on the choice), 128 or 256 pixels.  Estimated time, in units of one 32x128 block on a whole
  // compute unit: workgroups are handed out as residency slots free up, so the launch runs as
  // whole rounds of `slots` workgroups per unit plus a last partial round spread over the units; a
  // unit with one or two resident workgroups does not keep its MFMA pipes full.  The residency
  // figures follow the register use of the instances (wavefronts per SIMD: 8, 7, 5, 4 for 1..4 map
  // blocks x 128 pixels; 6, 4, 3, 2 for 256 pixels); a wrong figure costs speed, not correctness.
  static const int reg_slots[5][3] = {{0, 0, 0}, {0, 8, 6}, {0, 7, 4}, {0, 5, 3}, {0, 4, 2}};
  static const double fill[4] = {1.0, 0.7, 0.93, 0.97};  // MFMA rate with 1, 2, 3 workgroups on a unit
  // MFMA rate of an instance relative to what the round count alone predicts: measured time of every instance
  // against this estimate on the CaffeNet layers at batch 256 (conv3 / conv4 / conv5 forward and data gradient
  // for k = 3, conv2 whole and in two groups for k = 5), averaged per instance.  The 32 x 128 tile leads for
  // k = 3 (no vector ALU work is left in its step loop and eight workgroups share a compute unit).
  static const double rate3[5][3] = {{0, 0, 0}, {0, 1.023, 0.983}, {0, 0.985, 0.982}, {0, 0.967, 1.043}, {0, 1.0, 1.042}};
  static const double rate5[5][3] = {{0, 0, 0}, {0, 1.009, 1.017}, {0, 1.008, 0.975}, {0, 0.912, 1.022}, {0, 0.977, 1.03}};
  struct Candidate { DirectPlan plan; double cost; } cand[16];
  int ncand = 0;
  for (int l = 0; l < nlayouts; ++l) {
  const int nbands = layouts[l].nbands, wv = layouts[l].wv, pw = layouts[l].pw;
  const long ptot = (long)batch * nbands * wv * ho;  // the last band's columns past the right edge included
  if (ptot >= 2147483648L) continue;
  for (int tmb = 4; tmb >= 1; --tmb) {
    if (padded % (32 * tmb)) continue;
    const long tiles_m = padded / (32 * tmb);
    for (int tnb = 2; tnb >= 1; --tnb) {
      if (forced && forced != 10 * tmb + tnb) continue;
      const int bn = 128 * tnb;
      const int rows = (wv - 1 + bn - 1) / wv + 1, imgs = (wv * ho - 1 + bn - 1) / (wv * ho) + 1;
      const int pr = rows - 1 + (imgs - 1) * (ks - 1) + ks;
      const long patch = 2L * cp * pr * pw;
      const size_t lds =
          2 * (size_t)((2 * cp * 32 * tmb * ks * ks + 255) / 256 * 256 + (patch + 63) / 64 * 64) * sizeof(float);
      // the 7 x 7 instances ask for their LDS size (two map blocks of 49-tap slabs pass the default 64 KB)
      if (patch > 256L * kDirectPatchLoads || lds > (ks == 7 ? 80 : 64) * 1024 || (ks == 7 && tmb > 2)) continue;
      const long tiles = groups * tiles_m * ((ptot + bn - 1) / bn);
      long slots = (long)(160 * 1024 / lds);
      if (slots > reg_slots[tmb][tnb]) slots = reg_slots[tmb][tnb];
      const long full = tiles / (cus * slots), rest = tiles - full * cus * slots;
      const long last = (rest + cus - 1) / cus;
      const double work = tmb * tnb;
      const double cost = (full * slots * work / (slots < 4 ? fill[slots] : 1.0) +
                           last * work / (last < 4 ? fill[last] : 1.0)) /
                          (ks == 3 ? rate3[tmb][tnb] : rate5[tmb][tnb]);
      Candidate &c = cand[ncand++];
      c.plan.ks = ks; c.plan.tmb = tmb; c.plan.tnb = tnb; c.plan.cp = cp; c.plan.pw = pw; c.plan.pr = pr;
      c.plan.lds = lds; c.plan.wv = wv; c.plan.nbands = nbands;
      c.cost = cost;
    }
  }
  if (hp <= 64 && ncand) break;  // whole rows fit: no bands
  }
  if (ncand == 0) return false;
  const Candidate *pick = nullptr;
  for (int i = 0; i < ncand; ++i)
    if (!pick || cand[i].cost < pick->cost) pick = &cand[i];
  *pl = pick->plan;
  pl->tm16 = 0;
  return true;
}

template <int KS, int CP, int PW>
static int direct_launch_ks(const DirectArgs &g, const DirectPlan &pl, hipStream_t st) {
  dim3 grid(g.ntiles), block(256);
#define CCT_DIRECT_CASE(TMB, TNB)                                                                      \
  if (pl.tmb == TMB && pl.tnb == TNB) {                                                                \
    auto kern = conv_direct_kernel<KS, TMB, TNB, CP, PW>;                                              \
    if (pl.lds > 64 * 1024) {                                                                          \
      static LdsGrant grant;                                                                           \
      if (int rc = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc;                    \
    }                                                                                                  \
    hipLaunchKernelGGL(kern, grid, block, pl.lds, st, g);                                              \
    CCT_LAUNCH_CHECK();                                                                                \
    note_kernel("conv_direct_kernel<%d,%d,%d,%d,%d>", KS, TMB, TNB, CP, PW);                           \
    return 0;                                                                                          \
  }
  CCT_DIRECT_CASE(1, 1) CCT_DIRECT_CASE(2, 1) CCT_DIRECT_CASE(1, 2) CCT_DIRECT_CASE(2, 2)
  if constexpr (KS < 7) {  // 7 x 7: at most two map blocks (the slabs of more do not fit beside the patch)
    CCT_DIRECT_CASE(3, 1) CCT_DIRECT_CASE(4, 1) CCT_DIRECT_CASE(3, 2) CCT_DIRECT_CASE(4, 2)
  }
#undef CCT_DIRECT_CASE
  return set_error(CCT_HIP_EINVAL, "conv_direct: no kernel instance for tile %dx%d", pl.tmb, pl.tnb);
}

template <int KS, int PW>
static int direct_launch16(const DirectArgs &g, const DirectPlan &pl, hipStream_t st) {
  dim3 grid(g.ntiles), block(256);
#define CCT_DIRECT16_CASE(TM16, TNB)                                                                   \
  if (pl.tm16 == TM16 && pl.tnb == TNB) {                                                              \
    hipLaunchKernelGGL((conv_direct16_kernel<KS, TM16, TNB, PW>), grid, block, pl.lds, st, g);         \
    CCT_LAUNCH_CHECK();                                                                                \
    note_kernel("conv_direct16_kernel<%d,%d,%d,%d>", KS, TM16, TNB, PW);                               \
    return 0;                                                                                          \
  }
  CCT_DIRECT16_CASE(1, 1) CCT_DIRECT16_CASE(3, 1) CCT_DIRECT16_CASE(5, 1)
  CCT_DIRECT16_CASE(1, 2) CCT_DIRECT16_CASE(3, 2) CCT_DIRECT16_CASE(5, 2)
#undef CCT_DIRECT16_CASE
  return set_error(CCT_HIP_EINVAL, "conv_direct: no 16-row kernel instance for %d row blocks", pl.tm16);
}

// Phase store of a strided layer's data gradient (see DirectArgs::ss)
struct DirectShuffle {
  int s, hs, pad, d;
};

// `kc` channels and `mtot` maps PER GROUP; with groups > 1 the tensors hold groups * kc channels and
// groups * mtot maps per image and `wt` holds the groups' slab buffers one after another.
static int conv_direct(const float *wt, const float *src, float *dst, const float *bias, int relu, int batch, int kc,
                       int mtot, int hs, int ks, int pad, size_t src_img_stride, size_t dst_img_stride,
                       const float *mask = nullptr, const DirectShuffle *shuffle = nullptr, int groups = 1) {
  DirectPlan pl;
  CCT_REQUIRE(groups >= 1, "conv_direct: groups must be positive");
  CCT_REQUIRE(direct_plan(batch, kc, mtot, hs, ks, pad, &pl, groups),
              "conv_direct: geometry not covered (k=%d pad=%d size=%d)", ks, pad, hs);
  CCT_REQUIRE(!shuffle || pl.tm16, "conv_direct: the phase store needs the 16-row kernel");
  CCT_REQUIRE(!shuffle || groups == 1, "conv_direct: the phase store takes one group");
  DirectArgs g;
  g.ss = g.shs = g.spad = g.sd = 0;
  if (shuffle) {
    g.ss = shuffle->s; g.shs = shuffle->hs; g.spad = shuffle->pad; g.sd = shuffle->d;
    CCT_REQUIRE((double)batch * shuffle->d * shuffle->hs * shuffle->hs < 1073741824.0,
                "conv_direct: phase-store tensor too large");
  }
  g.wt = wt; g.src = src; g.dst = dst; g.bias = bias; g.relu = relu; g.mask = mask;
  g.batch = batch; g.kc = kc; g.mtot = mtot; g.hs = hs; g.pad = pad;
  g.ho = hs + 2 * pad - ks + 1;
  {
    const size_t dense_src = (size_t)groups * kc * hs * hs, dense_dst = (size_t)groups * mtot * g.ho * g.ho;
    if (!src_img_stride) src_img_stride = dense_src;
    if (!dst_img_stride) dst_img_stride = dense_dst;
    CCT_REQUIRE(src_img_stride >= dense_src && dst_img_stride >= dense_dst, "conv_direct: image stride smaller than an image");
    CCT_REQUIRE((double)batch * src_img_stride < 536870912.0 && (double)batch * dst_img_stride < 2147483648.0,
                "conv_direct: strided tensor too large for 32-bit byte offsets");
    g.src_img_stride = (uint32_t)src_img_stride;
    g.dst_img_stride = (uint32_t)dst_img_stride;
  }
  g.hp = g.ho + ks - 1;
  g.pr = pl.pr;
  g.nsteps = pl.tm16 ? (kc + 3) / 4 : (kc + 2 * pl.cp - 1) / (2 * pl.cp);
  CCT_REQUIRE((uintptr_t)wt % 16 == 0, "conv_direct: slab buffer must be 16-byte aligned");
  g.slab_stride = direct_padded_maps(mtot) * ks * ks;
  g.wv = pl.wv; g.nbands = pl.nbands; g.vpix = (uint32_t)(pl.wv * g.ho);
  g.ptot = (uint32_t)((long)batch * pl.nbands * g.vpix);
  g.tiles_m = pl.tm16 ? 1u : (uint32_t)((mtot + 32 * pl.tmb - 1) / (32 * pl.tmb));
  const uint32_t bn = 128 * pl.tnb;
  g.groups = groups;
  g.tiles_per_group = g.tiles_m * ((g.ptot + bn - 1) / bn);
  g.ntiles = g.tiles_per_group * (uint32_t)groups;
  g.wt_group_floats = (uint32_t)(direct_padded_channels(kc) * g.slab_stride);
  g.div_ho = make_fastdiv((uint32_t)g.ho);
  g.div_ho2 = make_fastdiv((uint32_t)(g.ho * g.ho));
  g.div_hp = make_fastdiv((uint32_t)g.hp);
  g.div_pr = make_fastdiv((uint32_t)g.pr);
  g.div_wv = make_fastdiv((uint32_t)g.wv);
  g.div_vpix = make_fastdiv(g.vpix);
  g.div_nbands = make_fastdiv((uint32_t)g.nbands);
  g.cs = g.pr * pl.pw + 16;
  g.div_cs = make_fastdiv((uint32_t)g.cs);
  hipStream_t st = ctx().stream;
  if (pl.tm16) {
    if (ks == 5)
      return pl.pw == 16 ? direct_launch16<5, 16>(g, pl, st)
                         : pl.pw == 32 ? direct_launch16<5, 32>(g, pl, st) : direct_launch16<5, 64>(g, pl, st);
    return pl.pw == 16 ? direct_launch16<3, 16>(g, pl, st)
                       : pl.pw == 32 ? direct_launch16<3, 32>(g, pl, st) : direct_launch16<3, 64>(g, pl, st);
  }
  if (ks == 7)
    return pl.pw == 16   ? direct_launch_ks<7, 1, 16>(g, pl, st)
           : pl.pw == 32 ? direct_launch_ks<7, 1, 32>(g, pl, st)
                         : direct_launch_ks<7, 1, 64>(g, pl, st);
  if (ks == 5)
    return pl.pw == 16   ? direct_launch_ks<5, 1, 16>(g, pl, st)
           : pl.pw == 32 ? direct_launch_ks<5, 1, 32>(g, pl, st)
                         : direct_launch_ks<5, 1, 64>(g, pl, st);
  return pl.pw == 16   ? direct_launch_ks<3, 2, 16>(g, pl, st)
         : pl.pw == 32 ? direct_launch_ks<3, 2, 32>(g, pl, st)
                       : direct_launch_ks<3, 2, 64>(g, pl, st);
}


// ---------------------------------------------------------------------------------------------
// Weight gradient without the lowered matrix:
//   dW[oo][c][kr][kc] = sum_{img,r,x} dout[img][oo][r][x] * src[img][c][r-pad+kr][x-pad+kc]
// as a GEMM with M = output maps, N = (c,kr,kc) columns and the contraction over output pixels.
//
// A workgroup of W wavefronts (W = 4..8) owns BM = 32*W maps x BN = 32*TB columns of dW and a range
// of contraction steps; wavefront w holds rows 32w..32w+31 for all TB column blocks.  One step is
// output row y of an image pair: MFMA lanes 0-31 take pixel (img0, y, x), lanes 32-63 pixel
// (img0+1, y, x), x = 0..ho-1.  Per step the workgroup stages, straight from global memory into
// LDS (global_load_lds, two LDS stages, one barrier per step):
//   * the dout slab [BM][ast]: words 0..ho-1 of a row = row y of img0, ho..2ho-1 = row y of img0+1
//     (ast odd, so the 32 rows a wavefront reads hit 32 banks).  The slab is filled as one flat run
//     of 64-word chunks with per-lane source offsets that are fixed for the whole tile;
//   * for the NCH channels its columns touch, the KS source rows under output row y of both
//     images, zero-padded ([NCH][2*KS][PWS]); every word is rewritten every step, out-of-image
//     words as zeros (out-of-range buffer loads).  PWS = KS and the channel stride = KS*KS (mod 32) make a
//     wavefront's 32 consecutive (c,kr,kc) columns read 32 different banks.
// Each lane's fragment addresses are base + x, so the loop over x only bumps offsets; fragments of
// the next two x are requested while the MFMAs of the current two run.  Partial sums of the step
// ranges go to a workspace and are added in a fixed order by direct_reduce_kernel (run-to-run
// identical results).
struct WgradArgs {
  const float *dout;   // [batch][o][ho][ho]
  const float *src;    // [batch][d][hs][hs]
  float *out;          // [splits][o][ncols]
  float *out_bias;     // [splits][o] bias-gradient partial sums, or null
  int batch, o, d, hs, ho, pad;
  int ncols;           // d * KS * KS
  int ast;             // floats between rows of the staged dout slab (odd)
  int bm;              // maps per workgroup = 32 * wavefronts
  int a_floats;        // slab floats per stage, multiple of 64
  int stage;           // floats per LDS stage
  int steps_total, steps_per_split;  // a step = (image pair, output row)
  uint32_t dout_img_stride, src_img_stride;  // floats between images (channel-slice views)
  uint32_t tiles_m, tiles_n, ntiles, nblocks;
  FastDiv div_ho, div_ast;
  // channel groups of a grouped convolution, all in this launch (o, d, ncols are PER GROUP): group q reads maps
  // q*o .. of dout and channels q*d .. of src and writes block q of the [splits][groups][o][ncols] partial sums;
  // ntiles = groups * tiles_per_group
  int groups;
  uint32_t tiles_per_group;
};

template <int KS, int PW>
struct WgradStrides {
  static constexpr int PWS = PW + KS;                                    // >= padded width; == KS (mod 32) for PW = 32
  static constexpr int RAW = 2 * KS * PWS;                               // two images' rows
  static constexpr int PCH = RAW + ((KS * KS - RAW) % 32 + 32) % 32;     // >= RAW, == KS*KS (mod 32)
};

constexpr int kWgradSlabLoads = 33;  // 64-word chunks of the dout slab per wavefront: ast/2 <= 32.5

template <int KS, int TB, int PW>
__global__ __launch_bounds__(512) void conv_direct_wgrad_kernel(const WgradArgs g) {
  constexpr int KK = KS * KS, BN = 32 * TB;
  constexpr int PWS = WgradStrides<KS, PW>::PWS, PCH = WgradStrides<KS, PW>::PCH;
  constexpr int NCH = (BN - 1) / KK + 2;                 // channels a column tile can touch
  constexpr int BSZ = (NCH * PCH + 63) / 64 * 64;        // patch floats per stage
  constexpr int NBL = (BSZ + 255) / 256;                 // source loads per lane per step (4 wavefronts)
  constexpr int NAL = kWgradSlabLoads;
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // known to be wave-uniform
  const int nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t z = flat / g.ntiles;
  uint32_t id = flat - z * g.ntiles;
  const uint32_t grp = g.groups > 1 ? id / g.tiles_per_group : 0u;  // workgroup-uniform
  id -= grp * g.tiles_per_group;
  const uint32_t tm = id / g.tiles_n, tn = id - tm * g.tiles_n;  // column tiles of one row tile run together
  const int m0 = tm * g.bm, n0 = tn * BN, ch0 = n0 / KK;
  const int s_beg = z * g.steps_per_split, s_end = min(g.steps_total, s_beg + g.steps_per_split);
  const int ho2 = g.ho * g.ho, hs2 = g.hs * g.hs;

  // ---- dout slab: chunk k of this wavefront covers slab words (k*nwaves + wave)*64 + lane ----
  const int a_chunks = g.a_floats >> 6;
  uint32_t aoff[NAL];   // source offset from the step base (img0, map m0, row y)
  uint32_t a_second = 0;  // bit k: the word belongs to the second image of the pair
#pragma unroll
  for (int k = 0; k < NAL; ++k) {
    const uint32_t e = (uint32_t)((k * nwaves + wave) * 64 + lane);
    const uint32_t m = fdiv(e, g.div_ast), i = e - m * g.ast;
    const uint32_t map = min((uint32_t)m0 + m, (uint32_t)g.o - 1) - m0;  // rows past the last map: any valid one
    uint32_t off = map * ho2;
    if (i < (uint32_t)g.ho) {
      off += i;
    } else if (i < 2u * g.ho) {
      off += g.dout_img_stride + (i - g.ho);
      a_second |= 1u << k;
    }
    aoff[k] = off * 4u;  // bytes; pad words and words past the slab read word 0 of a valid row
  }

  // ---- source patches: element e = pass*nthreads + tid of the dense [NCH][PCH] array ----
  uint32_t boff[NBL];  // source offset from the step base (img0, channel ch0, row y - pad)
  uint32_t bmeta[NBL]; // bits 0-3: patch row within the image (0..KS-1); bit 4: second image; bit 5: statically valid
#pragma unroll
  for (int k = 0; k < NBL; ++k) {
    const uint32_t e = (uint32_t)(k * nthreads + tid);
    const uint32_t ch = e / PCH, rem = e - ch * PCH;
    const uint32_t prow = rem / PWS, pcol = rem - prow * PWS;
    const uint32_t second = prow >= (uint32_t)KS ? 1u : 0u, kr = prow - second * KS;
    const int scol = (int)pcol - g.pad;
    const bool ok = e < (uint32_t)(NCH * PCH) && prow < 2u * KS && ch0 + (int)ch < g.d &&
                    (unsigned)scol < (unsigned)g.hs;
    boff[k] = ok ? (second * g.src_img_stride + ch * hs2 + kr * g.hs + (uint32_t)scol) * 4u : 0u;  // bytes
    bmeta[k] = kr | (second << 4) | ((ok ? 1u : 0u) << 5);
  }

  const rsrc_t a_rsrc = make_rsrc(g.dout + (size_t)grp * g.o * ho2), b_rsrc = make_rsrc(g.src + (size_t)grp * g.d * hs2);

// global -> LDS stage st for step s
#define CCT_WGRAD_ISSUE(s, st)                                                                    \
  do {                                                                                            \
    const uint32_t pair_ = fdiv((uint32_t)(s), g.div_ho);                                         \
    const int y_ = (s) - (int)pair_ * g.ho;                                                       \
    const int img0_ = 2 * (int)pair_;                                                             \
    const bool two_ = img0_ + 1 < g.batch;                                                        \
    float *sa_ = smem + (st) * g.stage;                                                           \
    const uint32_t ga_ = (uint32_t)(((size_t)img0_ * g.dout_img_stride + m0 * ho2 + y_ * g.ho) * 4); \
    /* odd batch, last image alone: the second image's half reads zeros */                        \
    const uint32_t second_ = two_ ? 0u : a_second;                                                \
    _Pragma("unroll") for (int k = 0; k < NAL; ++k) {                                             \
      if (k * nwaves + wave < a_chunks)                                                           \
        lds_dma4(a_rsrc, ((second_ >> k) & 1u) ? kOutOfRange : aoff[k], ga_,                      \
                 sa_ + (k * nwaves + wave) * 64);                                                 \
    }                                                                                             \
    float *sb_ = sa_ + g.a_floats;                                                                \
    const uint32_t gb_ = (uint32_t)(((size_t)img0_ * g.src_img_stride + ch0 * hs2) * 4);          \
    /* first patch row may lie above the image: that (negative) term goes into the lane offset, */ \
    /* whose sum is non-negative for every lane that passes the row test                        */ \
    const uint32_t row0_ = (uint32_t)((y_ - g.pad) * g.hs * 4);                                   \
    _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                             \
      const uint32_t mt_ = bmeta[k];                                                              \
      const int srow_ = y_ - g.pad + (int)(mt_ & 15u);                                            \
      const bool ok_ = (mt_ & 32u) && (unsigned)srow_ < (unsigned)g.hs && (two_ || !(mt_ & 16u)); \
      if (k * nthreads + wave * 64 < BSZ)                                                         \
        lds_dma4(b_rsrc, ok_ ? boff[k] + row0_ : kOutOfRange, gb_, sb_ + k * nthreads + wave * 64); \
    }                                                                                             \
  } while (0)

  // ---- fragment bases ----------------------------------------------------------------------
  const int abase = (wave * 32 + r) * g.ast + h * g.ho;
  int bbase[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = min(n0 + b * 32 + r, g.ncols - 1);
    const int c = col / KK, j = col - c * KK, kr = j / KS, kc = j - kr * KS;
    bbase[b] = g.a_floats + (c - ch0) * PCH + (h * KS + kr) * PWS + kc;
  }

  v16f acc[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
  // bias gradient: lane (r, h) adds up dout[map r][image h of every pair][every row][every x]
  float bsum = 0.0f;

  if (s_beg < s_end) {
    CCT_WGRAD_ISSUE(s_beg, 0);
    lds_dma_wait();
  }
  __syncthreads();

  const int quads = g.ho >> 2, rest = g.ho & 3;
  for (int s = s_beg; s < s_end; ++s) {
    const int cur = (s - s_beg) & 1;
    if (s + 1 < s_end) CCT_WGRAD_ISSUE(s + 1, cur ^ 1);
    const float *sa = smem + cur * g.stage + abase;
    const float *sb[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) sb[b] = smem + cur * g.stage + bbase[b];
    // fragment buffers: [buffer][x parity]; loads past ho stay inside the stage and are not used
    float fa[2][2], fb[2][2][TB];
#define CCT_WGRAD_FRAGS(buf, x)                                                                   \
  do {                                                                                            \
    fa[buf][0] = sa[(x)];                                                                         \
    fa[buf][1] = sa[(x) + 1];                                                                     \
    _Pragma("unroll") for (int b = 0; b < TB; ++b) {                                              \
      fb[buf][0][b] = sb[b][(x)];                                                                 \
      fb[buf][1][b] = sb[b][(x) + 1];                                                             \
    }                                                                                             \
  } while (0)
#define CCT_WGRAD_MFMA(buf, e)                                                                    \
  do {                                                                                            \
    bsum += fa[buf][e]; /* the dout fragment is also this lane's bias-gradient addend */         \
    _Pragma("unroll") for (int b = 0; b < TB; ++b)                                                \
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf][e], fb[buf][e][b], acc[b], 0, 0, 0); \
  } while (0)
// issue order of one x pair: an LDS read after every MFMA until the next pair's reads are out
#define CCT_WGRAD_ORDER()                                                                         \
  do {                                                                                            \
    _Pragma("unroll") for (int k2 = 0; k2 < TB + 1; ++k2) {                                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                          \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                          \
    }                                                                                             \
    __builtin_amdgcn_sched_group_barrier(0x008, TB - 1, 0);                                       \
    __builtin_amdgcn_sched_barrier(0);                                                            \
  } while (0)
    CCT_WGRAD_FRAGS(0, 0);
    for (int qd = 0; qd < quads; ++qd) {
      const int x = 4 * qd;
      CCT_WGRAD_FRAGS(1, x + 2);
      CCT_WGRAD_MFMA(0, 0);
      CCT_WGRAD_MFMA(0, 1);
      CCT_WGRAD_ORDER();
      CCT_WGRAD_FRAGS(0, x + 4);
      CCT_WGRAD_MFMA(1, 0);
      CCT_WGRAD_MFMA(1, 1);
      CCT_WGRAD_ORDER();
    }
    // remaining 0..3 columns; buffer 0 holds x = 4*quads and the one after it
    if (rest >= 1) CCT_WGRAD_MFMA(0, 0);
    if (rest >= 2) CCT_WGRAD_MFMA(0, 1);
    if (rest == 3) {
      CCT_WGRAD_FRAGS(1, 4 * quads + 2);
      CCT_WGRAD_MFMA(1, 0);
    }
#undef CCT_WGRAD_FRAGS
#undef CCT_WGRAD_MFMA
#undef CCT_WGRAD_ORDER
    lds_dma_wait();
    __syncthreads();
  }
#undef CCT_WGRAD_ISSUE

  if (g.out_bias && tn == 0) {
    // the two images of the pairs sit in the two lane halves; only the first column tile reports
    const float both = bsum + __shfl_xor(bsum, 32);
    const int row = m0 + wave * 32 + r;
    if (h == 0 && row < g.o) g.out_bias[((size_t)z * g.groups + grp) * g.o + row] = both;
  }
  float *out = g.out + ((size_t)z * g.groups + grp) * g.o * g.ncols;
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = n0 + b * 32 + r;
    if (col >= g.ncols) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wave * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < g.o) out[(size_t)row * g.ncols + col] = acc[b][v];
    }
  }
}


// The same computation with the output size, the wavefront count and hence every trip count known
// at compile time (the AlexNet/CaffeNet shapes; 3 x 3 layers with 7-, 14- and 28-pixel outputs, 5 x 5 layers with
// 14- and 28-pixel outputs): the whole step
// is one straight line of code, so
// the loads of the next step are spread between the MFMAs of this one instead of forming a phase
// of their own.  Differences from the generic kernel: each wavefront stages its own 32 rows of the
// dout slab (private, padded to whole 64-word loads), and the prefetch is unconditional -- the
// last step of a range re-fetches itself into the idle stage.
// With WN > 1 the workgroup is a W x WN grid of wavefronts: W row blocks times WN column groups of TB
// blocks each (192 maps = six row blocks then run as twelve wavefronts, three on every SIMD, instead
// of six wavefronts that leave two SIMDs half idle).
//
// ALDS: the dout rows go through LDS after all, fetched the way the patches are (4 bytes per lane straight into
// LDS, consecutive lanes on consecutive words of a row, rows packed HO words apart -- an odd stride, so the
// 32 maps of a wavefront fall on 32 banks).  A lane that fetches its own row touches a cache line of its own
// with every 16-byte load (64 lines per instruction); with few MFMAs per row -- three column blocks a
// wavefront, and both column groups fetching the same rows -- the address path of the texture unit is then
// busy for longer than the MFMAs of the step take.
template <int KS, int TB, int PW, int HO, int W, int WN = 1, bool ALDS = false>
__global__ __launch_bounds__(64 * W * WN) void conv_direct_wgrad_spec_kernel(const WgradArgs g) {
  constexpr int KK = KS * KS, BN = 32 * TB * WN, NT = 64 * W * WN;
  constexpr int PWS = WgradStrides<KS, PW>::PWS, PCH = WgradStrides<KS, PW>::PCH;
  constexpr int NCH = (BN - 1) / KK + 2;
  constexpr int BSZ = (NCH * PCH + NT - 1) / NT * NT;  // patch floats: whole passes
  constexpr int NBW = BSZ / NT;                        // patch loads per lane per step
  // dout never passes through LDS: lane (r, h) of a wavefront is the only reader of row y of map r
  // of image h, so it fetches that row itself, as NQD 16-byte buffer loads (runs of four floats;
  // the last run starts at HO - 4 and overlaps its neighbour when HO is not a multiple of 4) one
  // step ahead, into registers.  LDS then holds the source patches only, which lets several
  // workgroups share a compute unit: their barriers fall at different times and the MFMA pipes
  // stay fed across them.
  constexpr int NQD = (HO + 3) / 4;
  // ALDS: one image's 32 * W rows of HO words take NAI loads of 4 bytes per lane (whole passes), image 0 then
  // image 1, behind the patches of the stage
  constexpr int NAI = (32 * W * HO + NT - 1) / NT, AIMG = NAI * NT;
  constexpr int NAW = ALDS ? 2 * NAI : NQD;      // dout loads per lane per step
  constexpr int STAGE = BSZ + (ALDS ? 2 * AIMG : 0);
  constexpr int NQ = (HO + 1) / 2;                // x pairs per step
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = WN == 1 ? 0 : wave_id / W, wave = wave_id - wn * W;  // column group, row block
  const int r = lane & 31, h = lane >> 5;
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t z = flat / g.ntiles;
  uint32_t id = flat - z * g.ntiles;
  const uint32_t grp = g.groups > 1 ? id / g.tiles_per_group : 0u;  // workgroup-uniform
  id -= grp * g.tiles_per_group;
  const uint32_t tm = id / g.tiles_n, tn = id - tm * g.tiles_n;
  const int m0 = tm * (32 * W), n0 = tn * BN, ch0 = n0 / KK;
  const int s_beg = z * g.steps_per_split, s_end = min(g.steps_total, s_beg + g.steps_per_split);
  constexpr int ho2 = HO * HO;
  const int hs2 = g.hs * g.hs;

  // byte offset of this lane's dout row within (image pair, first map of the tile, row y)
  const uint32_t avoff =
      ((min((uint32_t)(m0 + wave * 32 + r), (uint32_t)g.o - 1) - m0) * ho2 + h * g.dout_img_stride) * 4u;
  // ALDS: byte offset of word k * NT + tid of an image's rows within (image, first map of the tile, row y)
  uint32_t aoff[ALDS ? NAI : 1];
  if constexpr (ALDS) {
#pragma unroll
    for (int k = 0; k < NAI; ++k) {
      const uint32_t e = (uint32_t)(k * NT + tid), m = e / HO, x = e - m * HO;
      aoff[k] = (m < 32u * W && m0 + (int)m < g.o) ? (m * ho2 + x) * 4u : kOutOfRange;
    }
  }
  const int abase = h * AIMG + (wave * 32 + r) * HO;  // this lane's row within the staged dout rows
  uint32_t boff[NBW], bmeta[NBW];
#pragma unroll
  for (int k = 0; k < NBW; ++k) {
    const uint32_t e = (uint32_t)(k * NT + tid);
    const uint32_t ch = e / PCH, rem = e - ch * PCH;
    const uint32_t prow = rem / PWS, pcol = rem - prow * PWS;
    const uint32_t second = prow >= (uint32_t)KS ? 1u : 0u, kr = prow - second * KS;
    const int scol = (int)pcol - g.pad;
    const bool ok = e < (uint32_t)(NCH * PCH) && prow < 2u * KS && ch0 + (int)ch < g.d &&
                    (unsigned)scol < (unsigned)g.hs;
    boff[k] = ok ? (second * g.src_img_stride + ch * hs2 + kr * g.hs + (uint32_t)scol) * 4u : kOutOfRange;
    bmeta[k] = kr + 8u * second;
  }
  // the patch descriptor starts `pad` rows ahead of the tensor (never read there: those rows fail the row test)
  const rsrc_t a_rsrc = make_rsrc(g.dout + (size_t)grp * g.o * ho2),
               b_rsrc = make_rsrc(g.src + (size_t)grp * g.d * hs2 - (ptrdiff_t)g.pad * g.hs);
  const rsrc_t a_none = make_rsrc_empty(g.dout);  // every load through it is out of range: zeros

  int bbase[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = min(n0 + (wn * TB + b) * 32 + r, g.ncols - 1);
    const int c = col / KK, j = col - c * KK, kr = j / KS, kc = j - kr * KS;
    bbase[b] = (c - ch0) * PCH + (h * KS + kr) * PWS + kc;
  }

  v16f acc[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
  // bias gradient: lane (r, h) adds up dout[map r][image h of every pair][every row][every x]
  float bsum = 0.0f;

  // The step loop is unrolled by two: the stage a step reads, P, and the stage its loads fill, P ^ 1, are
  // compile-time constants, so LDS addresses are fixed registers plus immediates and the lane-fetched dout rows
  // of the two stages are two register sets, never copied.  Whatever moves with the step (image pair, row) is
  // in the SCALAR offset of a load; a lane's own offset never changes, and what is left per patch load is the
  // test whether its source row exists (compare + select).  Vector ALU instructions and MFMAs of one SIMD do not
  // overlap, so every one of them taken out of the loop is four cycles returned to the MFMA pipe.
  struct StepScalars {
    uint32_t ga, gb, norows;
    bool two;
  };
  auto scalars_of = [&](int s) {
    StepScalars c;
    const uint32_t pair = fdiv((uint32_t)s, g.div_ho);
    const int y = s - (int)pair * HO;
    const int img0 = 2 * (int)pair;
    c.two = img0 + 1 < g.batch;
    c.ga = (uint32_t)(((size_t)img0 * g.dout_img_stride + m0 * ho2 + y * HO) * 4);
    // (the patch descriptor starts `pad` rows ahead of the tensor: row y + kr of it is source row y - pad + kr)
    c.gb = (uint32_t)(((size_t)img0 * g.src_img_stride + ch0 * hs2 + y * g.hs) * 4);
    // kernel rows kr whose source row y - pad + kr exists
    const int lo = max(0, g.pad - y), hi = min(KS - 1, g.hs - 1 + g.pad - y);
    const uint32_t one = hi >= lo ? ((2u << hi) - (1u << lo)) : 0u;
    c.norows = ~(one | (c.two ? one << 8 : 0u));
    return c;
  };
  f4 abuf[2][NQD];  // the dout row this lane fetched itself, per stage
#pragma unroll
  for (int k = 0; k < NQD; ++k) abuf[0][k] = abuf[1][k] = f4{0.f, 0.f, 0.f, 0.f};
  // dout loads of the step described by c, into stage st (IN: the step is an interior one)
#define CCT_WSPEC_A(k, st, c)                                                                     \
  do {                                                                                            \
    if constexpr (ALDS) {                                                                         \
      /* loads NAI .. 2 NAI - 1 are the second image's: all zeros when the pair has only one */   \
      if ((k) < NAI)                                                                              \
        lds_dma4(a_rsrc, aoff[(k) % NAI], c.ga, smem + (st) * STAGE + BSZ + (k) * NT + wave_id * 64); \
      else                                                                                        \
        lds_dma4(c.two ? a_rsrc : a_none, aoff[(k) % NAI], c.ga + g.dout_img_stride * 4u,         \
                 smem + (st) * STAGE + BSZ + (k) * NT + wave_id * 64);                            \
    } else {                                                                                      \
      abuf[st][(k) % NQD] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(         \
          a_rsrc, (!h || c.two) ? avoff : kOutOfRange,                                            \
          c.ga + ((k) + 1 < NQD ? 16u * (k) : 4u * (HO - 4)), 0));                                \
    }                                                                                             \
  } while (0)
#define CCT_WSPEC_B(k, st, c)                                                                     \
  do {                                                                                            \
    /* bmeta[k]: kernel row of a first-image lane, 8 + kernel row of a second-image lane; bit  */  \
    /* bmeta[k] of c.norows says that this row does not exist in the step, which moves the     */  \
    /* offset out of range (two vector instructions: bit-field extract, shift-or)              */  \
    lds_dma4(b_rsrc, boff[k] | (((c.norows >> bmeta[k]) & 1u) << 31), c.gb,                       \
             smem + (st) * STAGE + (k) * NT + wave_id * 64);                                      \
  } while (0)

  const bool do_bias = g.out_bias && tn == 0 && wn == 0;  // wave-uniform
  if (s_beg < s_end) {
    const StepScalars c0 = scalars_of(s_beg);
#pragma unroll
    for (int k = 0; k < NAW; ++k) CCT_WSPEC_A(k, 0, c0);
#pragma unroll
    for (int k = 0; k < NBW; ++k) CCT_WSPEC_B(k, 0, c0);
    lds_dma_wait();
  }
  __syncthreads();

  // fragment addresses per stage: patch columns of this lane's TB blocks, and its staged dout row
  int bb[2][TB], ab[2];
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    bb[0][b] = bbase[b];
    bb[1][b] = bbase[b] + STAGE;
    // (kept as a register of its own: seen as bb[0][b] + constant, it would be re-added before every read --
    // the paired LDS read reaches only 255 words beyond its address register)
    asm volatile("" : "+v"(bb[1][b]));
  }
  ab[0] = BSZ + abase;
  ab[1] = STAGE + BSZ + abase;
  asm volatile("" : "+v"(ab[1]));

  // one step: MFMAs on stage P, loads of the step described by c into stage P ^ 1
  auto step = [&](auto stage_c, const StepScalars &c) {
    constexpr int P = decltype(stage_c)::value, N = P ^ 1;
    float fa[2][2], fb[2][2][TB];
    // this lane's dout row: staged, or fetched by the lane during the previous step (pixel x is component
    // x % 4 of run x / 4, or of the overlapping last run)
#define CCT_WSPEC_AVAL(x)                                                                         \
  (ALDS ? smem[ab[P] + (x)]                                                                       \
        : ((x) < 4 * (NQD - 1) ? abuf[P][(x) / 4][(x) % 4] : abuf[P][NQD - 1][((x) - (HO - 4)) & 3]))
#define CCT_WSPEC_FRAGS(buf, x)                                                                   \
  do {                                                                                            \
    fa[buf][0] = CCT_WSPEC_AVAL(x);                                                               \
    fa[buf][1] = (x) + 1 < HO ? CCT_WSPEC_AVAL((x) + 1) : 0.0f;                                   \
    _Pragma("unroll") for (int b = 0; b < TB; ++b) {                                              \
      fb[buf][0][b] = smem[bb[P][b] + (x)];                                                       \
      fb[buf][1][b] = smem[bb[P][b] + (x) + 1];                                                   \
    }                                                                                             \
  } while (0)
    // bias gradient: only the wavefronts that report it add up their dout row (in pixel order), in one
    // block ahead of the MFMAs; the others carry no additions (when every wavefront made them, between
    // its MFMAs, they cost the benchmark shape's fifteen column tiles 1.8 %)
    if (do_bias) {
#pragma unroll
      for (int x = 0; x < HO; ++x) bsum += CCT_WSPEC_AVAL(x);
    }
    CCT_WSPEC_FRAGS(0, 0);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int cb = q & 1, nb = cb ^ 1;
      if (q + 1 < NQ) CCT_WSPEC_FRAGS(nb, 2 * q + 2);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (2 * q + e < HO) {
#pragma unroll
          for (int b = 0; b < TB; ++b)
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][e], fb[cb][e][b], acc[b], 0, 0, 0);
        }
      }
      // this pair's share of the next step's loads (all of them within the first NQI pairs, so that the
      // last ones have landed by the barrier)
      constexpr int NQI = (NQ * 5 + 7) / 8;
      const int qi = q < NQI ? q : NQI, qj = q + 1 < NQI ? q + 1 : NQI;
      const int a_lo = qi * NAW / NQI, a_hi = qj * NAW / NQI;
      const int b_lo = qi * NBW / NQI, b_hi = qj * NBW / NQI;
#pragma unroll
      for (int k = 0; k < NAW; ++k)
        if (k >= a_lo && k < a_hi) CCT_WSPEC_A(k, N, c);
#pragma unroll
      for (int k = 0; k < NBW; ++k)
        if (k >= b_lo && k < b_hi) CCT_WSPEC_B(k, N, c);
      // issue order: LDS reads of the next pair first, one per MFMA, then the global loads
      {
        constexpr int NM = 2 * TB;
        const int nr = (q + 1 < NQ) ? TB + (ALDS ? 1 : 0) : 0;
        const int nv = (a_hi - a_lo) + (b_hi - b_lo);
        const int nm = (2 * q + 1 < HO) ? NM : TB;
#pragma unroll
        for (int k2 = 0; k2 < NM; ++k2) {
          if (k2 < nm) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (k2 < nr) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          else if (k2 - nr < nv) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#undef CCT_WSPEC_FRAGS
#undef CCT_WSPEC_AVAL
    lds_dma_wait();
    __syncthreads();
  };
  // the loads of the last step of a range re-fetch that step into the idle stage
  auto run = [&](auto stage_c, int s) { step(stage_c, scalars_of(min(s + 1, s_end - 1))); };
  {
    int s = s_beg;
    for (; s + 1 < s_end; s += 2) {
      run(std::integral_constant<int, 0>{}, s);
      run(std::integral_constant<int, 1>{}, s + 1);
    }
    if (s < s_end) run(std::integral_constant<int, 0>{}, s);
  }
#undef CCT_WSPEC_A
#undef CCT_WSPEC_B

  if (do_bias) {
    // the two images of the pairs sit in the two lane halves; only the first column tile reports
    const float both = bsum + __shfl_xor(bsum, 32);
    const int row = m0 + wave * 32 + r;
    if (h == 0 && row < g.o) g.out_bias[((size_t)z * g.groups + grp) * g.o + row] = both;
  }
  float *out = g.out + ((size_t)z * g.groups + grp) * g.o * g.ncols;
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = n0 + (wn * TB + b) * 32 + r;
    if (col >= g.ncols) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wave * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < g.o) out[(size_t)row * g.ncols + col] = acc[b][v];
    }
  }
}

// dst[e] = sum_z ws[z][e] for e < n, and dst2[e - n] = sum_z ws2[z][e - n] for n <= e < n + n2;
// z ascending
__global__ __launch_bounds__(256) void direct_reduce_kernel(float *__restrict__ dst, const float *__restrict__ ws,
                                                            uint32_t n, float *__restrict__ dst2,
                                                            const float *__restrict__ ws2, uint32_t n2, int splits) {
  uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n + n2) return;
  if (e >= n) {
    e -= n; dst = dst2; ws = ws2; n = n2;
  }
  float s = 0.f;
  const float *p = ws + e;
  int z = 0;
  // eight partial sums in flight per lane; added in range order
  for (; z + 8 <= splits; z += 8, p += (size_t)8 * n) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[(size_t)j * n];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
  for (; z < splits; ++z, p += n) s += *p;
  dst[e] = s;
}

// The same sums for small results with many partial sums (LeNet-sized layers: 500 gradients, hundreds of
// step ranges), where one lane per element walks the ranges one after another and the launch is all
// latency: a workgroup takes 16 elements, its 16 lane groups each add up every 16th range (z = g, g + 16, ...,
// ascending), and lane group 0 adds the 16 group sums in ascending order.  A fixed order as well (run-to-run
// identical results), but another one than direct_reduce_kernel's, so a layer always takes the same kernel.
__global__ __launch_bounds__(256) void direct_reduce_small_kernel(float *__restrict__ dst, const float *__restrict__ ws,
                                                                  uint32_t n, float *__restrict__ dst2,
                                                                  const float *__restrict__ ws2, uint32_t n2,
                                                                  int splits) {
  __shared__ float part[16][17];
  const int el = threadIdx.x & 15, grp = threadIdx.x >> 4;
  uint32_t e = blockIdx.x * 16 + el;
  const bool live = e < n + n2;
  float s = 0.f;
  if (live) {
    const float *p;
    uint32_t stride;
    if (e >= n) { p = ws2 + (e - n); stride = n2; } else { p = ws + e; stride = n; }
    p += (size_t)grp * stride;
    int z = grp;
    for (; z + 48 < splits; z += 64, p += (size_t)64 * stride) {
      const float v0 = p[0], v1 = p[(size_t)16 * stride], v2 = p[(size_t)32 * stride], v3 = p[(size_t)48 * stride];
      s += v0; s += v1; s += v2; s += v3;
    }
    for (; z < splits; z += 16, p += (size_t)16 * stride) s += *p;
  }
  part[grp][el] = s;
  __syncthreads();
  if (grp == 0 && live) {
    float t = 0.f;
#pragma unroll
    for (int g2 = 0; g2 < 16; ++g2) t += part[g2][el];
    if (e >= n) dst2[e - n] = t;
    else dst[e] = t;
  }
}

int reduce_partial_sums(float *dst, const float *ws, uint32_t n, float *dst2, const float *ws2, uint32_t n2,
                        int splits, hipStream_t st) {
  if (n + n2 <= 8192 && splits >= 64)
    hipLaunchKernelGGL(direct_reduce_small_kernel, dim3((n + n2 + 15) / 16), dim3(256), 0, st, dst, ws, n, dst2, ws2,
                       n2, splits);
  else
    hipLaunchKernelGGL(direct_reduce_kernel, dim3((n + n2 + 255) / 256), dim3(256), 0, st, dst, ws, n, dst2, ws2, n2,
                       splits);
  CCT_LAUNCH_CHECK();
  return 0;
}

struct WgradPlan {
  int waves, tb, pw, ast, a_floats, stage;
  int wn;  // column groups of the workgroup's wavefront grid (specialised instances only, else 1)
  bool alds;  // specialised instances: the dout rows are staged in LDS
  bool spec;  // a compile-time specialised instance exists for this shape
  size_t lds;
};

static bool wgrad_plan(int batch, int d, int n, int ks, int pad, int o, WgradPlan *pl, int groups = 1) {
  if (ks != 3 && ks != 5) return false;
  const int ho = n + 2 * pad - ks + 1, hp = ho + ks - 1;
  if (pad < 0 || pad > ks - 1 || ho <= 0 || hp > 32 || batch <= 0 || d <= 0 || o <= 0) return false;
  // buffer loads address a tensor through 32-bit byte offsets
  if ((double)batch * groups * o * ho * ho >= 536870912.0 || (double)batch * groups * d * n * n >= 536870912.0 ||
      (double)groups * o * d * ks * ks >= 2147483648.0)
    return false;
  pl->pw = hp <= 16 ? 16 : 32;
  // wavefronts per workgroup (32 maps each): least padding of the map count, more wavefronts on ties
  // (8 and 4 first: they load the four SIMDs of a compute unit evenly)
  int best_w = 8;
  long best = -1;
  static const int wave_choices[5] = {8, 4, 6, 7, 5};
  for (int w : wave_choices) {
    const long padded = (long)((o + 32 * w - 1) / (32 * w)) * 32 * w;
    if (best < 0 || padded < best) { best = padded; best_w = w; }
  }
  pl->waves = best_w;
  if (const int forced = tuning().direct_waves) {  // tuning override
    if (forced >= 4 && forced <= 8) pl->waves = forced;
  }
  // column blocks per tile: least padding of the column count, wider tile on ties
  const long ncols = (long)d * ks * ks;
  // (narrow tiles re-read the dout slab for few MFMAs each: below 4 blocks only for small layers)
  int best_tb = 6;
  best = -1;
  for (int tb = 6; tb >= (ncols > 128 ? 4 : 1); --tb) {
    const long padded = (ncols + 32 * tb - 1) / (32 * tb) * 32 * tb;
    if (best < 0 || padded < best) { best = padded; best_tb = tb; }
  }
  {
    const int forced = tuning().direct_tb;  // tuning override
    if (forced >= 1 && forced <= 6) best_tb = forced;
  }
  pl->tb = best_tb;
  pl->ast = (2 * ho) | 1;
  pl->a_floats = (32 * pl->waves * pl->ast + 63) / 64 * 64;
  if ((pl->a_floats / 64 + pl->waves - 1) / pl->waves > kWgradSlabLoads) return false;
  const int pws = pl->pw + ks, raw = 2 * ks * pws;
  const int pch = raw + (((ks * ks - raw) % 32) + 32) % 32;  // WgradStrides<ks, pw>
  const int nch = (32 * pl->tb - 1) / (ks * ks) + 2;
  const int bsz = (nch * pch + 63) / 64 * 64;
  pl->stage = pl->a_floats + bsz;
  pl->spec = (ks == 5 && (ho == 27 || ho == 28 || ho == 14) && pl->pw == 32 && pl->tb == 5 &&
              (pl->waves == 4 || pl->waves == 8)) ||
             (ks == 3 && (ho == 13 || ho == 14 || ho == 7 || ho == 28) && pl->tb == 6 &&
              (pl->waves == 4 || pl->waves == 6 || pl->waves == 8));
  if (tuning().direct_nospec) pl->spec = false;  // tuning override
  pl->wn = 1;
  pl->alds = false;
  int nch_spec = nch;
  if (pl->spec) {
    // six row blocks: twelve wavefronts (six row blocks x two column groups of three blocks)
    if (pl->waves == 6) {
      pl->wn = 2;
      pl->tb = 3;
      nch_spec = (32 * pl->tb * pl->wn - 1) / (ks * ks) + 2;
    }
    // layout of conv_direct_wgrad_spec_kernel: dout stays out of LDS, patches in whole passes
    const int nt = 64 * pl->waves * pl->wn;
    pl->a_floats = 0;
    pl->stage = (nch_spec * pch + nt - 1) / nt * nt;
    // short rows: few MFMAs per row fetched, and a lane fetching its own row touches a cache line per load --
    // measured faster staged in LDS for the 3 x 3 instances on 7 to 14 pixel rows, slower on 27 and 28 pixel rows
    pl->alds = tuning().direct_alds == 1 || (tuning().direct_alds == 0 && ks == 3 && ho <= 14);
    if (pl->alds) pl->stage += 2 * ((32 * pl->waves * ho + nt - 1) / nt * nt);
  }
  // fragment loads may run a few words past the last patch row: the padding of the patch region
  // absorbs that, else a little slack is added
  const int tail_pad = pl->stage - pl->a_floats - nch_spec * pch;
  pl->lds = (size_t)(2 * pl->stage + (tail_pad >= 8 ? 0 : 16)) * sizeof(float);
  return pl->lds <= 160 * 1024;
}

template <int KS, int TB, int PW, int HO, int W, int WN, bool ALDS>
static int wgrad_launch_spec_as(const WgradArgs &g, const WgradPlan &pl, hipStream_t st) {
  auto kern = conv_direct_wgrad_spec_kernel<KS, TB, PW, HO, W, WN, ALDS>;
  static LdsGrant grant;
  if (int rc = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc;
  hipLaunchKernelGGL(kern, dim3(g.nblocks), dim3(64 * W * WN), pl.lds, st, g);
  CCT_LAUNCH_CHECK();
  note_kernel("conv_direct_wgrad_spec_kernel<%d,%d,%d,%d,%d,%d,%s>", KS, TB, PW, HO, W, WN, ALDS ? "true" : "false");
  return 0;
}
template <int KS, int TB, int PW, int HO, int W, int WN = 1>
static int wgrad_launch_spec(const WgradArgs &g, const WgradPlan &pl, hipStream_t st) {
  return pl.alds ? wgrad_launch_spec_as<KS, TB, PW, HO, W, WN, true>(g, pl, st)
                 : wgrad_launch_spec_as<KS, TB, PW, HO, W, WN, false>(g, pl, st);
}

// the 5 x 5 instances of one output size: 8 or 4 row blocks
template <int HO>
static int wgrad_launch_spec5(const WgradArgs &g, const WgradPlan &pl, hipStream_t st) {
  return pl.waves == 8 ? wgrad_launch_spec<5, 5, 32, HO, 8>(g, pl, st) : wgrad_launch_spec<5, 5, 32, HO, 4>(g, pl, st);
}

// the 3 x 3 instances of one output size: 8, 6 (as twelve wavefronts) or 4 row blocks
template <int HO, int PW = 16>
static int wgrad_launch_spec3(const WgradArgs &g, const WgradPlan &pl, hipStream_t st) {
  return pl.waves == 8   ? wgrad_launch_spec<3, 6, PW, HO, 8>(g, pl, st)
         : pl.waves == 6 ? wgrad_launch_spec<3, 3, PW, HO, 6, 2>(g, pl, st)
                         : wgrad_launch_spec<3, 6, PW, HO, 4>(g, pl, st);
}

template <int KS, int PW>
static int wgrad_launch(const WgradArgs &g, const WgradPlan &pl, hipStream_t st) {
  dim3 grid(g.nblocks), block(64 * pl.waves);
#define CCT_WGRAD_CASE(TB)                                                                              \
  if (pl.tb == TB) {                                                                                    \
    auto kern = conv_direct_wgrad_kernel<KS, TB, PW>;                                                   \
    static LdsGrant grant;                                                                              \
    if (int rc = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc;                       \
    hipLaunchKernelGGL(kern, grid, block, pl.lds, st, g);                                               \
    CCT_LAUNCH_CHECK();                                                                                 \
    note_kernel("conv_direct_wgrad_kernel<%d,%d,%d> waves=%d", KS, TB, PW, pl.waves);                   \
    return 0;                                                                                           \
  }
  CCT_WGRAD_CASE(1) CCT_WGRAD_CASE(2) CCT_WGRAD_CASE(3) CCT_WGRAD_CASE(4) CCT_WGRAD_CASE(5) CCT_WGRAD_CASE(6)
#undef CCT_WGRAD_CASE
  return set_error(CCT_HIP_EINVAL, "conv_direct wgrad: no kernel instance for %d column blocks", pl.tb);
}

// `d` channels and `o` maps PER GROUP; with groups > 1 the tensors hold groups * d channels and groups * o maps
// per image, dw is [groups][o][d][ks][ks] and db [groups][o].
static int conv_direct_wgrad(float *dw, float *db, const float *dout, const float *src, int batch, int d, int n,
                             int ks, int pad, int o, size_t src_img_stride, size_t dout_img_stride, int groups = 1) {
  WgradPlan pl;
  CCT_REQUIRE(groups >= 1, "conv_direct wgrad: groups must be positive");
  bool pairs = wgrad_plan(batch, d, n, ks, pad, o, &pl, groups);
  if (pairs && tuning().direct_wgrad_rows != 1) {
    // Image pairs pay off on short rows (a step of the one-image kernel is half as many MFMAs deep) and where a
    // compile-time instance exists.  Measured at 3 x 3, pairs against rows: 7-14 pixel rows 65-91 against 53-81
    // TFLOP/s (129 against 70 with a compile-time instance), 16 pixels 61 against 78, 20-30 pixels 25-81 against
    // 61-101 (the generic image-pair kernel wants 128 maps per workgroup); compile-time instances at 28 pixels
    // 105-136 against 97-113, at 14 pixels 111-134 against 77-82, at 7 pixels 99-118 against 50-56.
    // At 5 x 5 a step holds 25 MFMAs per column block instead of 9 and pairs stay ahead for longer: 14-pixel
    // outputs 65-88 against 56-67, 16-20 pixels 72-86 against 68-82, 24-28 pixels 39-80 against 67-95 -- except
    // with 256 maps (eight wavefronts, 107 against 95); compile-time instances 96-125 at 14 pixels and 81-144 at 28.
    const int longest_pair_row = ks == 5 ? 24 : 17;
    const bool rows = tuning().direct_wgrad_rows == 2 ||
                      (!pl.spec && n + 2 * pad > longest_pair_row && !(ks == 5 && o >= 256));
    if (rows && conv_strided_wgrad_covers(batch, d * groups, n, ks, 1, pad, o * groups) &&
        conv_strided_wgrad_covers(batch, d, n, ks, 1, pad, o))
      pairs = false;
  }
  if (!pairs) {
    // rows too long for the image-pair kernels: the one-image-per-step kernel, if its patch holds them,
    // group by group on channel slices
    CCT_REQUIRE(conv_strided_wgrad_covers(batch, d * groups, n, ks, 1, pad, o * groups) &&
                    conv_strided_wgrad_covers(batch, d, n, ks, 1, pad, o),
                "conv_direct wgrad: geometry not covered (k=%d pad=%d size=%d)", ks, pad, n);
    const int ho = n + 2 * pad - ks + 1;
    if (!src_img_stride) src_img_stride = (size_t)groups * d * n * n;
    if (!dout_img_stride) dout_img_stride = (size_t)groups * o * ho * ho;
    for (int q = 0; q < groups; ++q)
      if (int rc = conv_strided_wgrad(dw + (size_t)q * o * d * ks * ks, db ? db + (size_t)q * o : nullptr,
                                      dout + (size_t)q * o * ho * ho, src + (size_t)q * d * n * n, batch, d, n, ks, 1,
                                      pad, o, src_img_stride, dout_img_stride))
        return rc;
    return 0;
  }
  WgradArgs g;
  g.dout = dout; g.src = src;
  g.batch = batch; g.o = o; g.d = d; g.hs = n; g.pad = pad;
  g.ho = n + 2 * pad - ks + 1;
  g.ncols = d * ks * ks;
  {
    const size_t dense_src = (size_t)groups * d * n * n, dense_dout = (size_t)groups * o * g.ho * g.ho;
    if (!src_img_stride) src_img_stride = dense_src;
    if (!dout_img_stride) dout_img_stride = dense_dout;
    CCT_REQUIRE(src_img_stride >= dense_src && dout_img_stride >= dense_dout,
                "conv_direct wgrad: image stride smaller than an image");
    CCT_REQUIRE((double)batch * src_img_stride < 536870912.0 && (double)batch * dout_img_stride < 536870912.0,
                "conv_direct wgrad: strided tensor too large for 32-bit byte offsets");
    g.src_img_stride = (uint32_t)src_img_stride;
    g.dout_img_stride = (uint32_t)dout_img_stride;
  }
  g.ast = pl.ast; g.bm = 32 * pl.waves; g.a_floats = pl.a_floats; g.stage = pl.stage;
  g.steps_total = ((batch + 1) / 2) * g.ho;
  g.tiles_m = (uint32_t)((o + g.bm - 1) / g.bm);
  g.tiles_n = (uint32_t)((g.ncols + 32 * pl.tb * pl.wn - 1) / (32 * pl.tb * pl.wn));
  g.groups = groups;
  g.tiles_per_group = g.tiles_m * g.tiles_n;
  g.ntiles = g.tiles_per_group * (uint32_t)groups;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  // workgroups resident per compute unit: LDS and wavefront slots (two per SIMD is plenty here)
  int per_cu = (int)((160 * 1024) / pl.lds);
  if (per_cu > 8 / (pl.waves * pl.wn)) per_cu = 8 / (pl.waves * pl.wn);
  if (per_cu < 1) per_cu = 1;
  int splits = (int)((long)per_cu * cus / g.ntiles);
  if (tuning().direct_splits > 0) splits = tuning().direct_splits;  // tuning override
  if (splits < 1) splits = 1;
  if (splits > g.steps_total) splits = g.steps_total;
  g.steps_per_split = (g.steps_total + splits - 1) / splits;
  splits = (g.steps_total + g.steps_per_split - 1) / g.steps_per_split;
  g.nblocks = g.ntiles * (uint32_t)splits;
  g.div_ho = make_fastdiv((uint32_t)g.ho);
  g.div_ast = make_fastdiv((uint32_t)g.ast);
  const size_t n_out = (size_t)groups * o * g.ncols;  // all groups: dw is one contiguous [groups][o][ncols] block
  const int o_all = groups * o;
  if (splits > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)splits * (n_out + (db ? o_all : 0)) * sizeof(float), &ws);
    if (rc) return rc;
    g.out = (float *)ws;
    g.out_bias = db ? g.out + (size_t)splits * n_out : nullptr;
  } else {
    g.out = dw;
    g.out_bias = db;
  }
  hipStream_t st = ctx().stream;
  int rc;
  if (pl.spec && ks == 5)
    rc = g.ho == 27 ? wgrad_launch_spec5<27>(g, pl, st)
         : g.ho == 28 ? wgrad_launch_spec5<28>(g, pl, st)
                      : wgrad_launch_spec5<14>(g, pl, st);
  else if (pl.spec)
    rc = g.ho == 13 ? wgrad_launch_spec3<13>(g, pl, st)
         : g.ho == 14 ? wgrad_launch_spec3<14>(g, pl, st)
         : g.ho == 28 ? wgrad_launch_spec3<28, 32>(g, pl, st)
                      : wgrad_launch_spec3<7>(g, pl, st);
  else if (ks == 5) rc = pl.pw == 16 ? wgrad_launch<5, 16>(g, pl, st) : wgrad_launch<5, 32>(g, pl, st);
  else rc = pl.pw == 16 ? wgrad_launch<3, 16>(g, pl, st) : wgrad_launch<3, 32>(g, pl, st);
  if (rc) return rc;
  if (splits > 1) {
    const uint32_t n2 = db ? (uint32_t)o_all : 0u;
    if (int rc2 = reduce_partial_sums(dw, g.out, (uint32_t)n_out, db, g.out_bias, n2, splits, st)) return rc2;
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Data gradient of a STRIDED layer (stride S, kernel K) as a stride-1 convolution of the output
// gradient.  Write an input coordinate (in the zero-padded image) as i = S*I + pi: the taps that
// reach it are u = pi + S*a, a = 0 .. ceil(K/S) - 1, from output row I - a.  So each of the S*S
// (row phase, column phase) sub-images of every input channel is a small stride-1 convolution of
// the output gradient with its own KA x KA filter (KA = ceil(K/S), zero where pi + S*a >= K):
//   V[(c,pi,pj)][I][J] = sum_{m,a,b} w[m][c][pi + S*a][pj + S*b] * dout[m][I - a][J - b]
// which is conv_direct16_kernel's sum with d*S*S output maps, contraction over the layer's output
// maps, padding KA - 1 and reversed filters; the kernel's store puts V back at
// [c][S*I + pi - pad][S*J + pj - pad].  It replaces the gradient remap, the data-gradient GEMM, its
// (k*k*d) x (m*m*b) result and the lifting of ConvolutionBridge::backward.
//
// Slab buffer for it: wt[m][vm][u*KA + v] = w[m][c][pi + S*(KA-1-u)][pj + S*(KA-1-v)] with
// vm = (c*S + pi)*S + pj, zero for taps past the filter and for padding maps / channels.
__global__ __launch_bounds__(256) void strided_dgrad_slab_kernel(float *__restrict__ wt, const float *__restrict__ w,
                                                                 int n_o, int n_d, int ks, int stride, int ka,
                                                                 int p_m, uint32_t total, FastDiv div_kk,
                                                                 FastDiv div_m) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int kk = ka * ka, s2 = stride * stride;
  const uint32_t mv = fdiv(e, div_kk), t = e - mv * kk;
  const uint32_t m = fdiv(mv, div_m), vm = mv - m * p_m;
  float val = 0.f;
  if (m < (uint32_t)n_o && vm < (uint32_t)(n_d * s2)) {
    const int c = vm / s2, rem = vm - c * s2, pi = rem / stride, pj = rem - pi * stride;
    const int u = t / ka, v = t - u * ka;
    const int uu = pi + stride * (ka - 1 - u), vv = pj + stride * (ka - 1 - v);
    if (uu < ks && vv < ks) val = w[(((size_t)m * n_d + c) * ks + uu) * ks + vv];
  }
  wt[e] = val;
}

// KA of a (kernel size, stride) pair the phase decomposition covers: 3 or 5, or 0
static int strided_dgrad_ka(int ks, int stride) {
  if (stride < 2 || ks < stride) return 0;
  const int taps = (ks + stride - 1) / stride;
  return taps <= 3 ? 3 : taps <= 5 ? 5 : 0;
}

static bool strided_dgrad_plan(int batch, int d, int n, int ks, int stride, int pad, int o, DirectPlan *pl) {
  const int ka = strided_dgrad_ka(ks, stride);
  if (!ka || batch <= 0 || d <= 0 || o <= 0 || pad < 0 || pad >= ks || n + 2 * pad < ks) return false;
  const int ho = (n + 2 * pad - ks) / stride + 1;
  if (tuning().direct_tile != 0 && tuning().direct_tile != 161 && tuning().direct_tile != 162) return false;
  if ((double)batch * d * n * n >= 1073741824.0) return false;
  return direct_plan(batch, o, d * stride * stride, ho, ka, ka - 1, pl) && pl->tm16 > 0;
}

}  // namespace cct

using namespace cct;

static bool groups_divide(int groups, int depth, int num_outputs) {
  return groups >= 1 && depth > 0 && num_outputs > 0 && depth % groups == 0 && num_outputs % groups == 0;
}

extern "C" int cct_hip_conv_direct_supported_grouped(int batch, int depth, int n, int k, int stride, int padding,
                                                     int num_outputs, int groups) {
  if (stride != 1 || !groups_divide(groups, depth, num_outputs) || ensure_init() != 0) return 0;
  DirectPlan pl;
  const int m = n + 2 * padding - k + 1;
  const int dg = depth / groups, og = num_outputs / groups;
  // forward: channels = depth, maps = outputs, source n, pad p; data gradient: channels = outputs,
  // maps = depth, source m, pad k-1-p
  WgradPlan wp;
  return direct_plan(batch, dg, og, n, k, padding, &pl, groups) &&
                 direct_plan(batch, og, dg, m, k, k - 1 - padding, &pl, groups) &&
                 (wgrad_plan(batch, dg, n, k, padding, og, &wp, groups) ||
                  (conv_strided_wgrad_covers(batch, dg, n, k, 1, padding, og) &&
                   conv_strided_wgrad_covers(batch, depth, n, k, 1, padding, num_outputs)))
             ? 1
             : 0;
}

extern "C" int cct_hip_conv_direct_supported(int batch, int depth, int n, int k, int stride, int padding,
                                             int num_outputs) {
  return cct_hip_conv_direct_supported_grouped(batch, depth, n, k, stride, padding, num_outputs, 1);
}

extern "C" size_t cct_hip_conv_direct_slab_floats_grouped(int num_outputs, int depth, int k, int for_data_gradient,
                                                          int groups) {
  if (k <= 0 || !groups_divide(groups, depth, num_outputs)) return 0;
  const int og = num_outputs / groups, dg = depth / groups;
  const int n_c = for_data_gradient ? og : dg, n_m = for_data_gradient ? dg : og;
  return (size_t)groups * direct_padded_channels(n_c) * direct_padded_maps(n_m) * k * k;
}

extern "C" size_t cct_hip_conv_direct_slab_floats(int num_outputs, int depth, int k, int for_data_gradient) {
  return cct_hip_conv_direct_slab_floats_grouped(num_outputs, depth, k, for_data_gradient, 1);
}

extern "C" int cct_hip_conv_direct_slabs_grouped(float *slabs, const float *model, int num_outputs, int depth, int k,
                                                 int for_data_gradient, int groups) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(k > 0 && groups_divide(groups, depth, num_outputs), "conv_direct_slabs: bad dimensions");
  CCT_REQUIRE(slabs != model, "conv_direct_slabs: in-place use");
  const int og = num_outputs / groups, dg = depth / groups;
  const size_t total = cct_hip_conv_direct_slab_floats(og, dg, k, for_data_gradient);  // per group
  CCT_REQUIRE(total * groups < (1ull << 31), "conv_direct_slabs: model too large");
  // forward slabs: [depth][outputs][k*k]; data-gradient slabs: [outputs][depth][k*k] reversed; one such
  // buffer per group, one after another
  const int n_c = for_data_gradient ? og : dg, n_m = for_data_gradient ? dg : og;
  const int p_m = direct_padded_maps(n_m);
  hipLaunchKernelGGL(direct_slab_kernel, dim3((uint32_t)((total + 255) / 256), (uint32_t)groups), dim3(256), 0,
                     ctx().stream, slabs, model, n_c, n_m, p_m, (uint32_t)total, k * k, for_data_gradient ? 1 : 0,
                     make_fastdiv((uint32_t)(k * k)), make_fastdiv((uint32_t)p_m));
  CCT_LAUNCH_CHECK();
  return 0;
}

extern "C" int cct_hip_conv_direct_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                                         int for_data_gradient) {
  return cct_hip_conv_direct_slabs_grouped(slabs, model, num_outputs, depth, k, for_data_gradient, 1);
}

extern "C" int cct_hip_conv_direct_forward_grouped(float *output, const float *input, const float *slabs,
                                                   const float *bias, int batch, int depth, int n, int k,
                                                   int padding, int num_outputs, size_t input_image_stride,
                                                   size_t output_image_stride, int relu, int groups) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(groups_divide(groups, depth, num_outputs), "conv_direct_forward: groups must divide both depths");
  if (batch <= 0) return 0;
  return conv_direct(slabs, input, output, bias, relu != 0, batch, depth / groups, num_outputs / groups, n, k,
                     padding, input_image_stride, output_image_stride, nullptr, nullptr, groups);
}

extern "C" int cct_hip_conv_direct_forward(float *output, const float *input, const float *slabs,
                                           const float *bias, int batch, int depth, int n, int k, int padding,
                                           int num_outputs, size_t input_image_stride, size_t output_image_stride,
                                           int relu) {
  return cct_hip_conv_direct_forward_grouped(output, input, slabs, bias, batch, depth, n, k, padding, num_outputs,
                                             input_image_stride, output_image_stride, relu, 1);
}

extern "C" int cct_hip_conv_direct_backward_data_grouped(float *input_grad, const float *output_grad,
                                                         const float *slabs, int batch, int depth, int n, int k,
                                                         int padding, int num_outputs, size_t input_image_stride,
                                                         size_t output_image_stride, const float *relu_data,
                                                         int groups) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(groups_divide(groups, depth, num_outputs), "conv_direct_backward_data: groups must divide both depths");
  if (batch <= 0) return 0;
  const int m = n + 2 * padding - k + 1;
  return conv_direct(slabs, output_grad, input_grad, nullptr, 0, batch, num_outputs / groups, depth / groups, m, k,
                     k - 1 - padding, output_image_stride, input_image_stride, relu_data, nullptr, groups);
}

extern "C" int cct_hip_conv_direct_backward_data(float *input_grad, const float *output_grad,
                                                 const float *slabs, int batch, int depth, int n, int k,
                                                 int padding, int num_outputs, size_t input_image_stride,
                                                 size_t output_image_stride) {
  return cct_hip_conv_direct_backward_data_grouped(input_grad, output_grad, slabs, batch, depth, n, k, padding,
                                                   num_outputs, input_image_stride, output_image_stride, nullptr, 1);
}

extern "C" int cct_hip_conv_direct_backward_data_relu(float *input_grad, const float *output_grad,
                                                      const float *slabs, int batch, int depth, int n, int k,
                                                      int padding, int num_outputs, size_t input_image_stride,
                                                      size_t output_image_stride, const float *relu_data) {
  CCT_REQUIRE(relu_data, "conv_direct_backward_data_relu: null activation tensor");
  return cct_hip_conv_direct_backward_data_grouped(input_grad, output_grad, slabs, batch, depth, n, k, padding,
                                                   num_outputs, input_image_stride, output_image_stride, relu_data, 1);
}

extern "C" int cct_hip_conv_direct_backward_weights_grouped(float *model_grad, float *bias_grad,
                                                            const float *output_grad, const float *input, int batch,
                                                            int depth, int n, int k, int padding, int num_outputs,
                                                            size_t input_image_stride, size_t output_image_stride,
                                                            int groups) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(batch > 0, "conv_direct_backward_weights: empty batch");
  CCT_REQUIRE(groups_divide(groups, depth, num_outputs), "conv_direct_backward_weights: groups must divide both depths");
  return conv_direct_wgrad(model_grad, bias_grad, output_grad, input, batch, depth / groups, n, k, padding,
                           num_outputs / groups, input_image_stride, output_image_stride, groups);
}

extern "C" int cct_hip_conv_direct_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                                    const float *input, int batch, int depth, int n, int k,
                                                    int padding, int num_outputs, size_t input_image_stride,
                                                    size_t output_image_stride) {
  return cct_hip_conv_direct_backward_weights_grouped(model_grad, bias_grad, output_grad, input, batch, depth, n, k,
                                                      padding, num_outputs, input_image_stride, output_image_stride, 1);
}

extern "C" int cct_hip_conv_strided_backward_data_supported(int batch, int depth, int n, int k, int stride,
                                                            int padding, int num_outputs) {
  if (ensure_init() != 0) return 0;
  DirectPlan pl;
  return strided_dgrad_plan(batch, depth, n, k, stride, padding, num_outputs, &pl) ? 1 : 0;
}

extern "C" size_t cct_hip_conv_strided_backward_data_slab_floats(int num_outputs, int depth, int k, int stride) {
  const int ka = strided_dgrad_ka(k, stride);
  if (!ka || num_outputs <= 0 || depth <= 0) return 0;
  return (size_t)direct_padded_channels(num_outputs) * direct_padded_maps(depth * stride * stride) * ka * ka;
}

extern "C" int cct_hip_conv_strided_backward_data_slabs(float *slabs, const float *model, int num_outputs, int depth,
                                                        int k, int stride) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(slabs && model && slabs != model, "conv_strided_backward_data_slabs: null or in-place argument");
  const int ka = strided_dgrad_ka(k, stride);
  CCT_REQUIRE(ka && num_outputs > 0 && depth > 0, "conv_strided_backward_data_slabs: kernel size %d with stride %d is not covered", k, stride);
  const size_t total = cct_hip_conv_strided_backward_data_slab_floats(num_outputs, depth, k, stride);
  CCT_REQUIRE(total < (1ull << 31), "conv_strided_backward_data_slabs: model too large");
  const int p_m = direct_padded_maps(depth * stride * stride);
  hipLaunchKernelGGL(strided_dgrad_slab_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx().stream,
                     slabs, model, num_outputs, depth, k, stride, ka, p_m, (uint32_t)total,
                     make_fastdiv((uint32_t)(ka * ka)), make_fastdiv((uint32_t)p_m));
  CCT_LAUNCH_CHECK();
  return 0;
}

extern "C" int cct_hip_conv_strided_backward_data(float *input_grad, const float *output_grad, const float *slabs,
                                                  int batch, int depth, int n, int k, int stride, int padding,
                                                  int num_outputs) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(input_grad && output_grad && slabs, "conv_strided_backward_data: null argument");
  if (batch <= 0) return 0;
  DirectPlan pl;
  CCT_REQUIRE(strided_dgrad_plan(batch, depth, n, k, stride, padding, num_outputs, &pl),
              "conv_strided_backward_data: geometry not covered (k=%d stride=%d pad=%d size=%d)", k, stride, padding, n);
  const int ka = strided_dgrad_ka(k, stride);
  const int ho = (n + 2 * padding - k) / stride + 1;
  // rows / columns past the last one any tap reaches (the layer's floor division left them over) get no
  // store from the kernel: their gradient is zero
  if (stride * (ho + ka - 1) - padding < n)
    if (int rc = cct_hip_sconstant_initialize(input_grad, (size_t)batch * depth * n * n, 0.0f)) return rc;
  const DirectShuffle sh = {stride, n, padding, depth};
  return conv_direct(slabs, output_grad, input_grad, nullptr, 0, batch, num_outputs, depth * stride * stride, ho, ka,
                     ka - 1, 0, 0, nullptr, &sh);
}
