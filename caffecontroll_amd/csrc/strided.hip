// Strided convolution (stride 2 or 4, e.g. AlexNet / CaffeNet conv1: 11x11, stride 4) as a direct
// contraction on the gfx950 matrix cores, without the lowered matrix in memory.
//
//   dst[img][m][y][x] = bias[m] + sum_{c,u,v} w[m][c][u][v] * src[img][c][S*y - pad + u][S*x - pad + v]
//
// (out-of-image source elements count as zero; dst is ho x ho, ho = (hs + 2*pad - KS) / S + 1).
// It replaces lower_cube + forward GEMM + output remap + bias of the lowering pipeline; the sums run
// in another order than the lowered GEMM, so results agree with it to fp32 rounding, not bit for bit.
//
// Mapping.  One workgroup (4 wavefronts) computes BM = 32*TMB output maps x 128 consecutive output
// pixels (numbered across the whole batch).  The contraction runs over (channel c, tap row u, tap
// pair w): v_mfma_f32_32x32x2_f32 takes tap v = 2w from lanes 0-31 and v = 2w+1 from lanes 32-63, the
// tap row being padded with one zero weight when KS is odd (K = kc*KS*(KS+1) instead of kc*KS*KS).
//   * Source patch, one channel at a time: the rows of the (virtually stacked, zero-padded) images
//     that the tile's pixels touch, each row stored SPLIT BY COLUMN PHASE: [phase j][X] holds padded
//     column S*X + j.  Pixel x then reads tap v at phase v % S, index x + v / S: consecutive lanes read
//     consecutive LDS words (no bank conflicts although the image is read with stride S), and the two
//     lane halves differ by exactly one phase, so every fragment is one ds_read at lane base + a
//     wave-uniform offset.  The gather happens in the global -> LDS transfer (4-byte buffer loads
//     straight into LDS, out-of-image elements arrive as zeros).
//   * Weights: per (channel, tap row) a [map][AST] block, AST = KS+1 (+1) floats, odd so that the 32
//     maps of a fragment fall into 32 banks; the slab buffer has that layout, so the block is copied
//     to LDS as is with 16-byte loads, two tap rows per step.
// Two LDS stages for both; one barrier per step (two tap rows = 2*VP*TMB MFMAs per wavefront); the
// next channel's patch is fetched in slices spread over the steps of the current channel.
//
// Bound: fp32 MFMA rate.  Algorithmic work 2 * mtot * batch*ho*ho * kc*KS*KS FLOP per call.
#include <cstdlib>
#include <type_traits>

#include "cct_common.h"
#include "mfma_common.h"

namespace cct {

struct StridedArgs {
  const float *wt;    // slab buffer [kc][KSP][mpad][AST], zero padding (see conv_strided_slab_kernel)
  const float *src;   // [batch][kc][hs][hs]
  float *dst;         // [batch][mtot][ho][ho]
  const float *bias;  // [mtot] or null
  int relu;           // epilogue clamps at zero (ReLU of the layer that follows, folded in)
  int batch, kc, mtot, mpad, hs, ho, pad;
  int hp;             // hs + 2*pad: rows (and columns) of a zero-padded source image
  int xw;             // phase width: ceil(hp / S) (+ room for the padded tap)
  int rs;             // S * xw: floats of one patch row
  int pr;             // patch rows of a tile, at most
  uint32_t ptot;      // batch * ho * ho
  uint32_t tiles_m, ntiles;
  FastDiv div_ho, div_ho2, div_hp, div_rs, div_xw;
};

constexpr int kStridedPatchLoads = 28;  // 4-byte source loads per lane per channel, at most (28 KB of patch)

template <int KS, int S, int TMB>
__global__ __launch_bounds__(256, 2) void conv_strided_kernel(const StridedArgs g) {
  constexpr int VP = (KS + 1) / 2;          // tap pairs per tap row
  constexpr int AST = (2 * VP) | 1;         // floats per map in a weight block (odd)
  constexpr int BM = 32 * TMB, BN = 128;
  constexpr int UPS = 2;                    // tap rows per step
  constexpr int NST = (KS + UPS - 1) / UPS; // steps per channel
  constexpr int KSP = NST * UPS;            // tap rows in the slab buffer (zero rows past KS)
  constexpr int UB4 = BM * AST / 4;         // 16-byte vectors of one tap row's weight block
  constexpr int WSZ = UPS * BM * AST;       // floats of weights per step
  constexpr int WSZP = (WSZ + 255) / 256 * 256;
  constexpr int NW4 = (WSZP / 4 + 255) / 256;  // 16-byte loads per lane per step
  constexpr int NPL = kStridedPatchLoads;
  constexpr int PSZ = NPL * 256;            // floats of one patch stage
  // patch loads issued in step st of a channel (for the next channel): all but the last step
  constexpr int NPS = (NPL + NST - 2) / (NST - 1);
  static_assert(BM * AST % 4 == 0, "weight blocks are copied in 16-byte vectors");
  static_assert(S == 2 || S == 4, "the two lane halves must sit one column phase apart");
  static_assert(NST >= 2, "at least two steps per channel");
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float *const smP = smem;                // two patch stages
  float *const smW = smem + 2 * PSZ;      // two weight stages

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;

  const uint32_t id = xcd_remap(blockIdx.x, g.ntiles);
  const uint32_t tn = id / g.tiles_m, tm = id - tn * g.tiles_m;
  const int m0 = tm * BM;
  const uint32_t p0 = tn * BN;
  const int ho2 = g.ho * g.ho;

  // first patch row: the virtual (stacked, padded) row under the first tap of the tile's first pixel
  const uint32_t img0 = fdiv(p0, g.div_ho2);
  const uint32_t y0 = fdiv(p0 - img0 * ho2, g.div_ho);
  const int r_lo = img0 * g.hp + S * y0;

  // ---- loader state ------------------------------------------------------------------------------
  uint32_t aoff[NW4];
#pragma unroll
  for (int i = 0; i < NW4; ++i) {
    const int e4 = tid + i * 256;
    const int ul = e4 / UB4, f = (e4 - ul * UB4) * 4;
    aoff[i] = ul < UPS ? (uint32_t)(ul * g.mpad * AST + f) * 4u : kOutOfRange;  // bytes
  }
  // patch element e = (patch row, phase, X): source = padded column S*X + phase of that virtual row
  uint32_t psrc[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const uint32_t e = tid + i * 256;
    const uint32_t prow = fdiv(e, g.div_rs), rem = e - prow * g.rs;
    const uint32_t ph = fdiv(rem, g.div_xw), X = rem - ph * g.xw;
    const uint32_t vr = r_lo + prow;
    const uint32_t img = fdiv(vr, g.div_hp);
    const int srow = (int)(vr - img * g.hp) - g.pad, scol = (int)(S * X + ph) - g.pad;
    const bool ok = prow < (uint32_t)g.pr && img < (uint32_t)g.batch && (unsigned)srow < (unsigned)g.hs &&
                    (unsigned)scol < (unsigned)g.hs;
    psrc[i] = ok ? ((img * g.kc * g.hs + srow) * g.hs + scol) * 4u : kOutOfRange;  // channel 0; bytes
  }
  const uint32_t c_step = (uint32_t)g.hs * g.hs * 4u;                  // bytes between channels of the source
  const uint32_t u_step = (uint32_t)g.mpad * AST * 4u;                 // bytes between tap rows of the slabs
  const rsrc_t a_rsrc = make_rsrc(g.wt + (size_t)m0 * AST), b_rsrc = make_rsrc(g.src);
  const int wave_elem0 = wave * 64;

// weights of step st of channel c -> weight stage ws (asynchronous)
#define CCT_STRIDED_ISSUE_W(c, st, ws)                                                          \
  do {                                                                                          \
    float *dst_ = smW + (ws) * WSZP;                                                            \
    const uint32_t ga_ = (uint32_t)((c) * KSP + (st) * UPS) * u_step;                           \
    _Pragma("unroll") for (int i = 0; i < NW4; ++i) {                                           \
      if (i * 256 + wave_elem0 < WSZP / 4)                                                      \
        lds_dma16(a_rsrc, (i * 256 + tid < WSZ / 4) ? aoff[i] : kOutOfRange, ga_,               \
                  dst_ + (i * 256 + wave_elem0) * 4);                                           \
    }                                                                                           \
  } while (0)
// loads [lo, hi) of the patch of channel c -> patch stage ps (asynchronous); channels past the last
// one fetch zeros
#define CCT_STRIDED_ISSUE_P(c, ps, lo, hi)                                                      \
  do {                                                                                          \
    float *dst_ = smP + (ps) * PSZ;                                                             \
    const bool real_ = (c) < g.kc;                                                              \
    const uint32_t gb_ = real_ ? (uint32_t)(c) * c_step : 0u;                                   \
    _Pragma("unroll") for (int i = 0; i < NPL; ++i) {                                           \
      if (i >= (lo) && i < (hi))                                                                \
        lds_dma4(b_rsrc, real_ ? psrc[i] : kOutOfRange, gb_, dst_ + i * 256 + wave_elem0);      \
    }                                                                                           \
  } while (0)

  // ---- fragment bases ----------------------------------------------------------------------------
  const int abase = r * AST + h;
  int bbase;
  {
    uint32_t p = p0 + wave * 32 + r;
    p = min(p, g.ptot - 1);
    const uint32_t img = fdiv(p, g.div_ho2);
    const uint32_t pix = p - img * ho2;
    const uint32_t y = fdiv(pix, g.div_ho), x = pix - y * g.ho;
    bbase = (int)(img * g.hp + S * y - r_lo) * g.rs + (int)x + h * g.xw;
  }

  v16f acc[TMB];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[a][e] = 0.0f;

  CCT_STRIDED_ISSUE_P(0, 0, 0, NPL);
  CCT_STRIDED_ISSUE_W(0, 0, 0);
  lds_dma_wait();
  __syncthreads();

  for (int c = 0; c < g.kc; ++c) {
    const float *pst = smP + (c & 1) * PSZ;
#pragma unroll
    for (int st = 0; st < NST; ++st) {
      const int t = c * NST + st;
      const float *wst = smW + (t & 1) * WSZP;
      // next step's weights (every wave finished reading that stage before the barrier that ended the
      // previous step); then this step's slice of the next channel's patch.  Loads complete in issue
      // order, so waiting until only the patch slice is outstanding means the weights have landed.
      const bool more = t + 1 < g.kc * NST;
      if (more) CCT_STRIDED_ISSUE_W(st + 1 < NST ? c : c + 1, st + 1 < NST ? st + 1 : 0, (t + 1) & 1);
      if (st < NST - 1) CCT_STRIDED_ISSUE_P(c + 1, (c + 1) & 1, st * NPS, (st + 1) * NPS < NPL ? (st + 1) * NPS : NPL);
      constexpr int NI = UPS * VP;  // contraction pairs of the step (those of tap rows past KS are skipped)
      float fa[2][TMB], fb[2];
#define CCT_STRIDED_FRAGS(buf, idx)                                                             \
  do {                                                                                          \
    const int ul_ = (idx) / VP, w_ = (idx) % VP, v_ = 2 * w_;                                   \
    const int u_ = st * UPS + ul_;                                                              \
    _Pragma("unroll") for (int a = 0; a < TMB; ++a)                                             \
        fa[buf][a] = wst[ul_ * BM * AST + abase + a * 32 * AST + v_];                           \
    fb[buf] = pst[bbase + u_ * g.rs + (v_ % S) * g.xw + v_ / S];                                \
  } while (0)
      // pairs of tap rows past the last one carry zero weights: skipped (st, idx are compile-time)
#define CCT_STRIDED_LIVE(idx) (st * UPS + (idx) / VP < KS)
      if (CCT_STRIDED_LIVE(0)) CCT_STRIDED_FRAGS(0, 0);
#pragma unroll
      for (int q = 0; q < NI; ++q) {
        const int cb = q & 1, nb = cb ^ 1;
        if (q + 1 < NI && CCT_STRIDED_LIVE(q + 1)) CCT_STRIDED_FRAGS(nb, q + 1);
        if (CCT_STRIDED_LIVE(q)) {
#pragma unroll
          for (int a = 0; a < TMB; ++a)
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][a], fb[cb], acc[a], 0, 0, 0);
        }
        // issue order: the LDS reads of the next pair go out between this pair's MFMAs
        if (CCT_STRIDED_LIVE(q)) {
#pragma unroll
          for (int k2 = 0; k2 < TMB; ++k2) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (k2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#undef CCT_STRIDED_FRAGS
#undef CCT_STRIDED_LIVE
      // weights of the next step have landed; at most this step's patch slice is still in flight
      // (after the last slice-carrying step: everything)
      if (st < NST - 2) __builtin_amdgcn_s_waitcnt(0x0F70 | NPS);
      else lds_dma_wait();
      __syncthreads();
    }
  }
#undef CCT_STRIDED_ISSUE_W
#undef CCT_STRIDED_ISSUE_P

  // ---- epilogue: accumulator register v of lane (r,h) is row 8*(v/4) + 4*h + v%4, column r ----
  const uint32_t p = p0 + wave * 32 + r;
  if (p >= g.ptot) return;
  const uint32_t img = fdiv(p, g.div_ho2);
  float *out = g.dst + (size_t)img * g.mtot * ho2 + (p - img * ho2);
  // the lane's bias values first, all loads in flight together (rows past the last map read a valid one)
  float bv[TMB][16];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int v = 0; v < 16; ++v) bv[a][v] = 0.f;
  if (g.bias) {
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) bv[a][v] = g.bias[min(m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4), g.mtot - 1)];
  }
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < g.mtot) {
        const float y = acc[a][v] + bv[a][v];
        out[(size_t)row * ho2] = (g.relu && !(y > 0.f)) ? 0.f : y;
      }
    }
}

// The same convolution for layers WITHOUT padding (conv1 of AlexNet / CaffeNet), with the source
// operand kept out of LDS altogether: the KS source elements under tap row u of a lane's pixel,
// src[img][c][S*y + u][S*x .. S*x + KS - 1], are contiguous in memory, so the lane fetches them
// itself (16-byte buffer loads, one step ahead; consecutive pixels -> consecutive 16-byte runs).
// A step covers two tap rows, whose 2*KS taps are paired in flattened order, so an odd kernel
// size wastes a tap only in the last step of a channel; the lane half picks the even or odd tap
// of each pair out of the registers.  LDS holds the weight blocks only, in three stages: the
// block of step g+2 is requested in the middle of step g, right after the one barrier of the
// step, and that barrier never falls on a stage switch, so the fragments of the first pairs of
// step g+1 are already on their way when step g ends and the matrix pipe does not drain.
struct StridedRegArgs {
  const float *wt;    // slab buffer [kc][NST][mpad][AST], zero padding (see conv_strided_step_slab_kernel)
  const float *src;   // [batch][kc][hs][hs]
  float *dst;         // [batch][mtot][ho][ho]
  const float *bias;  // [mtot] or null
  int relu;
  int batch, kc, mtot, mpad, hs, ho;
  uint32_t ptot, tiles_m, ntiles;
  FastDiv div_ho, div_ho2;
};

template <int N>
__device__ __forceinline__ void load_run(float (&dst)[N], rsrc_t r, uint32_t voff, uint32_t soff) {
  // N consecutive floats as 16-byte loads plus one shorter load for the tail
#pragma unroll
  for (int q = 0; q + 4 <= N; q += 4) {
    const f4 v = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(r, voff + 4u * q, soff, 0));
    dst[q] = v[0]; dst[q + 1] = v[1]; dst[q + 2] = v[2]; dst[q + 3] = v[3];
  }
  constexpr int T = N % 4, Q = N - T;
  if (T == 3) {
    typedef float f3 __attribute__((ext_vector_type(3)));
    const f3 v = __builtin_bit_cast(f3, __builtin_amdgcn_raw_buffer_load_b96(r, voff + 4u * Q, soff, 0));
    dst[Q] = v[0]; dst[Q + 1] = v[1]; dst[Q + 2] = v[2];
  } else if (T == 2) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = __builtin_bit_cast(f2, __builtin_amdgcn_raw_buffer_load_b64(r, voff + 4u * Q, soff, 0));
    dst[Q] = v[0]; dst[Q + 1] = v[1];
  } else if (T == 1) {
    dst[Q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff + 4u * Q, soff, 0));
  }
}

// s_waitcnt vmcnt(n) for an n that is a constant only after unrolling (the instruction takes an immediate)
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
  switch (n) {
#define CCT_VMCNT_CASE(N) case N: __builtin_amdgcn_s_waitcnt(0x0F70 | N); break;
    CCT_VMCNT_CASE(1) CCT_VMCNT_CASE(2) CCT_VMCNT_CASE(3) CCT_VMCNT_CASE(4) CCT_VMCNT_CASE(5)
    CCT_VMCNT_CASE(6) CCT_VMCNT_CASE(7) CCT_VMCNT_CASE(8) CCT_VMCNT_CASE(9) CCT_VMCNT_CASE(10)
    CCT_VMCNT_CASE(11) CCT_VMCNT_CASE(12) CCT_VMCNT_CASE(13) CCT_VMCNT_CASE(14) CCT_VMCNT_CASE(15)
#undef CCT_VMCNT_CASE
    default: lds_dma_wait(); break;
  }
}

template <int KS, int S, int TMB>
__global__ __launch_bounds__(256, 4) void conv_strided_reg_kernel(const StridedRegArgs g) {
  constexpr int BM = 32 * TMB, BN = 128;
  constexpr int UPS = 2;                      // tap rows per step
  constexpr int NST = (KS + UPS - 1) / UPS;   // steps per channel
  constexpr int NPF = (UPS * KS + 1) / 2;     // tap pairs of a full step
  constexpr int AST = (2 * NPF) | 1;          // floats per map in a step's weight block (odd)
  constexpr int WSZ = BM * AST;               // floats of weights per step
  constexpr int NW4 = (WSZ / 4 + 255) / 256;  // 16-byte loads per lane per step
  constexpr int WSZP = NW4 * 1024;            // floats of one stage: every lane issues every load
  constexpr int LPR = (KS + 3) / 4;           // source load instructions per tap row
  static_assert(WSZ % 4 == 0, "weight blocks are copied in 16-byte vectors");
  static_assert(UPS * LPR < 16, "the load counter of the mid-step wait is four bits wide here");
  extern __shared__ __attribute__((aligned(16))) float smem[];  // three weight stages

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31;
  const bool hi = lane >= 32;
  const int h = hi ? 1 : 0;

  const uint32_t id = xcd_remap(blockIdx.x, g.ntiles);
  const uint32_t tn = id / g.tiles_m, tm = id - tn * g.tiles_m;
  const int m0 = tm * BM;
  const uint32_t p0 = tn * BN;
  const int ho2 = g.ho * g.ho;
  const int nsteps = g.kc * NST;

  uint32_t aoff[NW4];
#pragma unroll
  for (int i = 0; i < NW4; ++i) {
    const int e4 = tid + i * 256;
    aoff[i] = e4 < WSZ / 4 ? (uint32_t)e4 * 16u : kOutOfRange;  // lanes past the block write zeros
  }
  const uint32_t step_bytes = (uint32_t)g.mpad * AST * 4u;  // bytes between the blocks of two steps
  const rsrc_t a_rsrc = make_rsrc(g.wt + (size_t)m0 * AST), b_rsrc = make_rsrc(g.src);
#define CCT_SREG_ISSUE_W(step, ws)                                                              \
  do {                                                                                          \
    float *dst_ = smem + (ws) * WSZP + wave * 256;                                              \
    const uint32_t ga_ = (uint32_t)(step) * step_bytes;                                         \
    _Pragma("unroll") for (int i = 0; i < NW4; ++i) lds_dma16(a_rsrc, aoff[i], ga_, dst_ + i * 1024); \
  } while (0)

  // this lane's pixel and the byte offset of the first source element under its first tap
  uint32_t p = p0 + wave * 32 + r;
  p = min(p, g.ptot - 1);
  const uint32_t img = fdiv(p, g.div_ho2);
  const uint32_t pix = p - img * ho2;
  const uint32_t y = fdiv(pix, g.div_ho), x = pix - y * g.ho;
  const uint32_t boff = ((img * g.kc * g.hs + S * y) * g.hs + S * x) * 4u;
  const uint32_t row_bytes = (uint32_t)g.hs * 4u, chan_bytes = (uint32_t)g.hs * g.hs * 4u;

  const int abase = r * AST + h;
  v16f acc[TMB];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[a][e] = 0.0f;

  // source runs of the rows of the coming step (raw) and of the current step (tap chosen by lane half)
  float nxt[UPS][KS], cur[NPF];
#pragma unroll
  for (int ul = 0; ul < UPS; ++ul)
    if (ul < KS) load_run<KS>(nxt[ul], b_rsrc, boff, (uint32_t)ul * row_bytes);
  CCT_SREG_ISSUE_W(0, 0);
  if (nsteps > 1) CCT_SREG_ISSUE_W(1, 1);
  lds_dma_wait();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  float fn[TMB];  // weight fragments of the coming pair
#pragma unroll
  for (int a = 0; a < TMB; ++a) fn[a] = smem[abase + a * 32 * AST];
  int rsg = 0;    // stage of the current step where the step count of a channel is no multiple of three

  for (int c = 0; c < g.kc; ++c) {
#pragma unroll
    for (int st = 0; st < NST; ++st) {
      const int sg = NST % 3 == 0 ? st % 3 : rsg;            // stage of this step
      const int sg1 = sg == 2 ? 0 : sg + 1, sg2 = sg == 0 ? 2 : sg - 1;  // of the next one, of the one after
      const float *wst = smem + sg * WSZP, *wnx = smem + sg1 * WSZP;
      const int live = (st + 1) * UPS <= KS ? UPS : KS - st * UPS;  // tap rows of this step
      const int ntap = live * KS, NP = (ntap + 1) / 2, H = NP / 2 > 0 ? NP / 2 : 1;
      // pick the even (lanes 0-31) or odd (lanes 32-63) tap of each pair; the tap past the last one is zero
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        const float even = nxt[(2 * q) / KS][(2 * q) % KS];
        const float odd = 2 * q + 1 < ntap ? nxt[(2 * q + 1) / KS][(2 * q + 1) % KS] : 0.0f;
        cur[q] = hi ? odd : even;
      }
      // the source rows of the step after this one: the next tap rows of this channel, or the first of the next channel
      const bool wrap = st + 1 == NST;
      const bool more = !wrap || c + 1 < g.kc;
      const int nst = wrap ? 0 : st + 1;
      const int nbl = ((nst + 1) * UPS <= KS ? UPS : KS - nst * UPS) * LPR;  // load instructions that fetch them
      if (more) {
        const uint32_t cb = (uint32_t)(wrap ? c + 1 : c) * chan_bytes;
#pragma unroll
        for (int ul = 0; ul < UPS; ++ul)
          if (nst * UPS + ul < KS) load_run<KS>(nxt[ul], b_rsrc, boff, cb + (uint32_t)(nst * UPS + ul) * row_bytes);
      }
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        float fc[TMB];
#pragma unroll
        for (int a = 0; a < TMB; ++a) fc[a] = fn[a];
        // fragments of the next pair: of this step, or the first of the next step (a stage that the
        // barrier of this step has already published; after the last step the values go unused)
#pragma unroll
        for (int a = 0; a < TMB; ++a)
          fn[a] = q + 1 < NP ? wst[abase + a * 32 * AST + 2 * (q + 1)] : wnx[abase + a * 32 * AST];
#pragma unroll
        for (int a = 0; a < TMB; ++a)
          acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(fc[a], cur[q], acc[a], 0, 0, 0);
#pragma unroll
        for (int k2 = 0; k2 < TMB; ++k2) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (q == H - 1) {
          // Middle of the step.  This wave's part of the next step's weight block was requested a
          // step ago, before the source rows just requested: wait for it alone, meet the other
          // waves (they are all past the previous step, whose stage is free now), request the block
          // of the step after the next.
          if (more) wait_vmcnt_upto(nbl);
          else lds_dma_wait();
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
          if (st + 2 < NST || c + 1 < g.kc) CCT_SREG_ISSUE_W(c * NST + st + 2, sg2);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (NST % 3 != 0) rsg = sg1;
    }
  }
#undef CCT_SREG_ISSUE_W

  // ---- epilogue: accumulator register v of lane (r,h) is row 8*(v/4) + 4*h + v%4, column r ----
  const uint32_t pe = p0 + wave * 32 + r;
  if (pe >= g.ptot) return;
  if (m0 + BM <= g.mtot) {
    // Every row of the tile exists (always, when the map count is a multiple of the tile: conv1's 96).  With a
    // contraction of only k*k*d = 363 the tile runs 183 MFMAs per channel, so the address arithmetic of 16 * TMB
    // stores per lane is a visible share of the kernel: here each store is one buffer store whose lane offset is
    // the same for all of them (row m0 + 4h at the lane's pixel) and whose row offset is a scalar; the bias comes in
    // as 16-byte loads of the four consecutive rows a lane holds per accumulator quarter.
    const rsrc_t o_rsrc = make_rsrc(g.dst);
    const uint32_t voff = (uint32_t)((((size_t)img * g.mtot + m0 + 4 * h) * ho2 + pix) * 4u);
    const uint32_t plane = (uint32_t)ho2 * 4u;
    f4 bq[TMB][4];
    if (g.bias) {
      const rsrc_t bias_rsrc = make_rsrc(g.bias);
#pragma unroll
      for (int a = 0; a < TMB; ++a)
#pragma unroll
        for (int qv = 0; qv < 4; ++qv)
          bq[a][qv] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(
                                                 bias_rsrc, 16u * h, (uint32_t)(m0 + a * 32 + 8 * qv) * 4u, 0));
    }
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float yv = acc[a][v];
        if (g.bias) yv += bq[a][v / 4][v % 4];
        if (g.relu) yv = (yv > 0.f) ? yv : 0.f;
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, yv), o_rsrc, voff,
                                              (uint32_t)(a * 32 + 8 * (v / 4) + (v % 4)) * plane, 0);
      }
    return;
  }
  float *out = g.dst + (size_t)img * g.mtot * ho2 + pix;
  float bv[TMB][16];
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int v = 0; v < 16; ++v) bv[a][v] = 0.f;
  if (g.bias) {
#pragma unroll
    for (int a = 0; a < TMB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) bv[a][v] = g.bias[min(m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4), g.mtot - 1)];
  }
#pragma unroll
  for (int a = 0; a < TMB; ++a)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < g.mtot) {
        const float yv = acc[a][v] + bv[a][v];
        out[(size_t)row * ho2] = (g.relu && !(yv > 0.f)) ? 0.f : yv;
      }
    }
}

// wt[((c*KSP + u)*mpad + m)*AST + j] = w[m][c][u][j] for m < n_m, u < ks, j < ks; zero elsewhere.
// One thread per element of the padded buffer.
__global__ __launch_bounds__(256) void conv_strided_slab_kernel(float *__restrict__ wt, const float *__restrict__ w,
                                                                int n_c, int n_m, int mpad, int ks, int ksp, int ast,
                                                                uint32_t total, FastDiv div_ast, FastDiv div_m,
                                                                FastDiv div_ksp) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const uint32_t t1 = fdiv(e, div_ast), j = e - t1 * ast;
  const uint32_t t2 = fdiv(t1, div_m), m = t1 - t2 * mpad;
  const uint32_t c = fdiv(t2, div_ksp), u = t2 - c * ksp;
  float v = 0.f;
  if (m < (uint32_t)n_m && u < (uint32_t)ks && j < (uint32_t)ks)
    v = w[(((size_t)m * n_c + c) * ks + u) * ks + j];
  wt[e] = v;
}

// Step-major slab buffer of the kernel without padding: the block of channel c, step st holds, for
// every map m, the taps of tap rows 2*st and 2*st+1 in flattened order,
// wt[((c*nst + st)*mpad + m)*ast + j] = w[m][c][2*st + j/ks][j%ks]; zero for maps, tap rows and j past the end.
__global__ __launch_bounds__(256) void conv_strided_step_slab_kernel(float *__restrict__ wt, const float *__restrict__ w,
                                                                     int n_c, int n_m, int mpad, int ks, int nst, int ast,
                                                                     uint32_t total, FastDiv div_ast, FastDiv div_m,
                                                                     FastDiv div_nst, FastDiv div_ks) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const uint32_t t1 = fdiv(e, div_ast), j = e - t1 * ast;
  const uint32_t t2 = fdiv(t1, div_m), m = t1 - t2 * mpad;
  const uint32_t c = fdiv(t2, div_nst), st = t2 - c * nst;
  const uint32_t ul = fdiv(j, div_ks), v = j - ul * ks, u = 2 * st + ul;
  float val = 0.f;
  if (m < (uint32_t)n_m && ul < 2 && u < (uint32_t)ks) val = w[(((size_t)m * n_c + c) * ks + u) * ks + v];
  wt[e] = val;
}

struct StridedPlan {
  int ks, s, tmb, vp, ast, ksp, mpad, xw, rs, pr;
  int nst, ast_step;  // step-major slab buffer (no padding): steps per channel, floats per map in a block
  size_t lds, lds_step;
};

// Chooses the instance for a geometry; false when the strided direct path does not cover it.
static bool strided_plan(int batch, int d, int n, int ks, int stride, int pad, int o, StridedPlan *pl) {
  if (!((ks == 11 && stride == 4) || (ks == 7 && stride == 2) || (ks == 5 && stride == 2) || (ks == 3 && stride == 2)))
    return false;
  if (batch <= 0 || d <= 0 || o <= 0 || pad < 0 || pad >= ks || n + 2 * pad < ks) return false;
  const int hp = n + 2 * pad, ho = (hp - ks) / stride + 1;
  // buffer loads address the tensors through 32-bit byte offsets
  if ((double)batch * d * n * n >= 536870912.0 || (double)batch * o * ho * ho >= 536870912.0) return false;
  pl->ks = ks; pl->s = stride;
  pl->vp = (ks + 1) / 2;
  pl->ast = (2 * pl->vp) | 1;
  pl->ksp = (ks + 1) / 2 * 2;
  pl->nst = (ks + 1) / 2;
  pl->ast_step = (2 * ((2 * ks + 1) / 2)) | 1;
  // output-map tile: least padding, larger tile on ties (instances: 1, 2, 3 row blocks)
  int best_t = 1;
  long best = -1;
  for (int t = 3; t >= 1; --t) {
    const long padded = (long)((o + 32 * t - 1) / (32 * t)) * 32 * t;
    if (best < 0 || padded < best) { best = padded; best_t = t; }
  }
  pl->tmb = best_t;
  pl->mpad = (o + 32 * best_t - 1) / (32 * best_t) * 32 * best_t;
  pl->xw = pl->rs = pl->pr = 0;
  pl->lds = 0;
  {
    const int nw4 = (32 * best_t * pl->ast_step / 4 + 255) / 256;
    pl->lds_step = (size_t)3 * nw4 * 1024 * sizeof(float);
  }
  if (pad == 0) return true;  // the lanes fetch the source themselves: no patch to fit
  // phase width: every phase holds the columns the taps can reach, the zero tap of an odd row included
  pl->xw = (ho - 1) + (2 * pl->vp - 1) / stride + 1;
  if (pl->xw < (hp + stride - 1) / stride) pl->xw = (hp + stride - 1) / stride;
  pl->rs = stride * pl->xw;
  // Rows a tile of 128 consecutive pixels can touch, in the virtual stack of padded images: from
  // the first tap row of its first pixel (image i, output row y) to the last tap row of its last
  // pixel (image i + di, output row y + dy): di*hp + S*dy + KS.  The pixel count bounds dy for every
  // di < batch: di*ho*ho + dy*ho + (x1 - x0) = 127 with x1 - x0 >= -(ho - 1).
  pl->pr = 0;
  for (int di = 0; di < batch && di * ho * ho <= 127 + (ho - 1) * (ho + 1); ++di) {
    const int room = 127 - di * ho * ho + ho - 1;
    const int dy = room >= 0 ? room / ho : -((-room + ho - 1) / ho);
    if (dy < -(ho - 1)) break;
    const int rows = di * hp + stride * (dy < ho - 1 ? dy : ho - 1) + ks;
    if (rows > pl->pr) pl->pr = rows;
  }
  if ((long)pl->pr * pl->rs > (long)kStridedPatchLoads * 256) return false;
  const int wszp = (2 * 32 * best_t * pl->ast + 255) / 256 * 256;
  pl->lds = (size_t)(2 * kStridedPatchLoads * 256 + 2 * wszp) * sizeof(float);
  return pl->lds <= 80 * 1024;
}

template <int KS, int S>
static int strided_launch(const StridedArgs &g, const StridedPlan &pl, hipStream_t st) {
  dim3 grid(g.ntiles), block(256);
  if (g.pad == 0) {
    // without padding every tap of every pixel lies inside the image: the lanes fetch the source themselves
    StridedRegArgs q;
    q.wt = g.wt; q.src = g.src; q.dst = g.dst; q.bias = g.bias; q.relu = g.relu;
    q.batch = g.batch; q.kc = g.kc; q.mtot = g.mtot; q.mpad = g.mpad; q.hs = g.hs; q.ho = g.ho;
    q.ptot = g.ptot; q.tiles_m = g.tiles_m; q.ntiles = g.ntiles; q.div_ho = g.div_ho; q.div_ho2 = g.div_ho2;
    const size_t lds = pl.lds_step;
#define CCT_STRIDED_REG_CASE(TMB)                                                               \
  if (pl.tmb == TMB) {                                                                          \
    hipLaunchKernelGGL((conv_strided_reg_kernel<KS, S, TMB>), grid, block, lds, st, q);         \
    CCT_LAUNCH_CHECK();                                                                         \
    note_kernel("conv_strided_reg_kernel<%d,%d,%d>", KS, S, TMB);                               \
    return 0;                                                                                   \
  }
    CCT_STRIDED_REG_CASE(1) CCT_STRIDED_REG_CASE(2) CCT_STRIDED_REG_CASE(3)
#undef CCT_STRIDED_REG_CASE
  }
#define CCT_STRIDED_CASE(TMB)                                                                   \
  if (pl.tmb == TMB) {                                                                          \
    auto kern = conv_strided_kernel<KS, S, TMB>;                                                \
    static LdsGrant grant;                                                                      \
    if (int rc = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc;               \
    hipLaunchKernelGGL(kern, grid, block, pl.lds, st, g);                                       \
    CCT_LAUNCH_CHECK();                                                                         \
    note_kernel("conv_strided_kernel<%d,%d,%d>", KS, S, TMB);                                   \
    return 0;                                                                                   \
  }
  CCT_STRIDED_CASE(1) CCT_STRIDED_CASE(2) CCT_STRIDED_CASE(3)
#undef CCT_STRIDED_CASE
  return set_error(CCT_HIP_EINVAL, "conv_strided: no kernel instance for %d row blocks", pl.tmb);
}


// ---------------------------------------------------------------------------------------------
// Weight gradient of a strided layer without the lowered matrix:
//   dW[m][c][u][v] = sum_{img,y,x} dout[img][m][y][x] * src[img][c][S*y - pad + u][S*x - pad + v]
// as a GEMM with M = output maps, N = (c,u,v) columns and the contraction over output pixels
// (it replaces the output-gradient remap and the weight-gradient GEMM against the lowered matrix,
// and with them the need to keep that matrix from the forward pass).
//
// A workgroup is a WM x WN grid of wavefronts and owns 32*WM maps x 32*TB*WN columns of dW and a
// range of contraction steps; wavefront (wm, wn) holds row block wm for the TB column blocks of
// column group wn.  One step is output row y of one image: MFMA lanes 0-31 take pixel x = 2q,
// lanes 32-63 pixel x = 2q + 1.  Per step the workgroup stages, straight from global memory into
// LDS (4-byte buffer loads into LDS, two stages, one barrier per step):
//   * the dout slab [32*WM][ast]: words 0..ho-1 of a row = row y of that map, zeros behind (ast odd:
//     the 32 rows a wavefront reads hit 32 banks);
//   * for the channels its columns touch, the KS source rows under output row y, zero-padded:
//     [channel][KS][pws]; pws = KS and the channel stride = KS*KS (mod 32), so a wavefront's 32
//     consecutive (c,u,v) columns read 32 different banks, and pixel x reads its row at S*x.
//     Every word is rewritten every step (out-of-image words arrive as zeros).
// Partial sums of the step ranges go to a workspace and are added in a fixed order
// (run-to-run identical results).  The bias gradient rides along: the dout fragments a wavefront
// of column group 0 feeds to the matrix cores are also summed per lane.
// Output rows too long for one step's slab and patch (images wider than some 60 pixels at stride 1) are taken in
// pieces of cw pixels: a step is then (image, row, piece), the piece's first pixel x0 moves both operands' scalar
// offsets, and what lies outside the image -- left of it in the first piece, right of it and past the row's end in
// the last -- is masked per lane by bit sets fixed at the start (the patch descriptor starts `pad` floats ahead
// of the tensor, so that every lane offset is non-negative).
//
// Bound: fp32 MFMA rate.  Algorithmic work 2 * o * batch*ho*ho * d*KS*KS FLOP per call.
struct StridedWgradArgs {
  const float *dout;   // [batch][o][ho][ho]
  const float *src;    // [batch][d][hs][hs]
  float *out;          // [splits][o][ncols]
  float *out_bias;     // [splits][o] bias-gradient partial sums, or null
  int batch, o, d, hs, ho, pad;
  int ncols;           // d * KS * KS
  int wm, wn;          // wavefront grid of a workgroup
  int nch;             // channels of the source patch
  int ast;             // floats between rows of the dout slab (odd)
  int a_floats, b_floats;  // slab / patch floats per stage, whole passes of the workgroup
  int nal, nbl;        // loads per lane per step: slab, patch
  int pws, pch;        // floats between patch rows / patch channels
  int nq2;             // groups of four pixels per step: ceil(cw / 4)
  int cw, nchunks;     // a long output row is taken in nchunks pieces of cw pixels (the last may be shorter); ho, 1 otherwise
  int steps_total, steps_per_split;  // a step = (image, output row, piece of the row)
  uint32_t dout_img_stride, src_img_stride;  // floats between images (channel-slice views of wider tensors)
  uint32_t tiles_m, tiles_n, ntiles, nblocks;
  FastDiv div_ho, div_ast, div_pch, div_pws, div_wm, div_nchunks;
};

constexpr int kSWgradSlabLoads = 16;   // per lane per step, at most
constexpr int kSWgradPatchLoads = 20;

template <int KS, int S, int TB>
__global__ __launch_bounds__(768) void conv_strided_wgrad_kernel(const StridedWgradArgs g) {
  constexpr int KK = KS * KS;
  constexpr int NAL = kSWgradSlabLoads, NBL = kSWgradPatchLoads;
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nthreads = blockDim.x, nwaves = nthreads >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int wni = (int)fdiv((uint32_t)wave, g.div_wm), wmi = wave - wni * g.wm;
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t z = flat / g.ntiles, id = flat - z * g.ntiles;
  const uint32_t tm = id / g.tiles_n, tn = id - tm * g.tiles_n;
  const int bm = 32 * g.wm;
  const int m0 = tm * bm, n0 = tn * (32 * TB * g.wn), ch0 = n0 / KK;
  const int s_beg = z * g.steps_per_split, s_end = min(g.steps_total, s_beg + g.steps_per_split);
  const int ho2 = g.ho * g.ho, hs2 = g.hs * g.hs;
  const int stage = g.a_floats + g.b_floats;

  // ---- dout slab: pass k of the workgroup covers slab words k*nthreads + tid ----
  const int x_last = (g.nchunks - 1) * g.cw;  // first pixel of a row's last piece
  const int tw = S * (g.cw - 1) + KS;         // source columns a piece touches
  uint32_t aoff[NAL];  // byte offset from (image, map m0, row y, pixel x0); kOutOfRange = a zero word
  uint32_t a_last = 0u, b_first = 0u, b_last = 0u;  // per load: the word exists in the last / first / last piece
#pragma unroll
  for (int k = 0; k < NAL; ++k) {
    const uint32_t e = (uint32_t)(k * nthreads + tid);
    const uint32_t m = fdiv(e, g.div_ast), i = e - m * g.ast;
    const bool ok = k < g.nal && m < (uint32_t)bm && m0 + (int)m < g.o && i < (uint32_t)g.cw;
    aoff[k] = ok ? (m * ho2 + i) * 4u : kOutOfRange;
    if (x_last + (int)i < g.ho) a_last |= 1u << k;  // the pixel exists in the last piece of a row
  }
  // ---- source patch: element e = k*nthreads + tid of the [nch][pch] array (rows of pws floats) ----
  uint32_t boff[NBL];               // byte offset from (image, channel ch0, row S*y - pad, column S*x0 - pad); kOutOfRange = never valid
  uint32_t brow[(NBL + 4) / 5];     // tap row of each element, six bits apiece
#pragma unroll
  for (int k = 0; k < (NBL + 4) / 5; ++k) brow[k] = 0u;
#pragma unroll
  for (int k = 0; k < NBL; ++k) {
    const uint32_t e = (uint32_t)(k * nthreads + tid);
    const uint32_t ch = fdiv(e, g.div_pch), rem = e - ch * g.pch;
    const uint32_t prow = fdiv(rem, g.div_pws), pcol = rem - prow * g.pws;
    const bool ok = k < g.nbl && ch < (uint32_t)g.nch && prow < (uint32_t)KS && ch0 + (int)ch < g.d &&
                    pcol < (uint32_t)tw;
    boff[k] = ok ? (ch * hs2 + prow * g.hs + pcol) * 4u : kOutOfRange;
    brow[k / 5] |= (ok ? prow : 0u) << (6 * (k % 5));
    if ((int)pcol >= g.pad) b_first |= 1u << k;                       // not left of the image in the first piece
    if (S * x_last + (int)pcol - g.pad < g.hs) b_last |= 1u << k;     // not right of it in the last piece
  }
  const rsrc_t a_rsrc = make_rsrc(g.dout), b_rsrc = make_rsrc(g.src - g.pad);
  if (g.nchunks == 1) {
    // a row in one piece: what the first and the last piece leave out is left out of every step
#pragma unroll
    for (int k = 0; k < NAL; ++k)
      if (!((a_last >> k) & 1u)) aoff[k] = kOutOfRange;
#pragma unroll
    for (int k = 0; k < NBL; ++k)
      if (!((b_first & b_last) >> k & 1u)) boff[k] = kOutOfRange;
  }
  // (image, output row, piece) of the next step to fetch, kept as counters (steps are fetched in order)
  int nx_img, nx_y, nx_piece;
  {
    const uint32_t rowid = fdiv((uint32_t)s_beg, g.div_nchunks);
    nx_piece = s_beg - (int)rowid * g.nchunks;
    nx_img = (int)fdiv(rowid, g.div_ho);
    nx_y = (int)rowid - nx_img * g.ho;
  }

// global -> LDS stage st for the next step.  A step whose k source rows lie inside the image -- nearly every one --
// needs next to no per-lane work: every load is a fixed lane offset plus a scalar offset, and only the first and
// the last piece of a row in several pieces mark the words they lack (two instructions per load).  (Issuing these
// loads in batches between the MFMAs of the current step instead of all at its start measured 3-10 % slower.)
#define CCT_SWGRAD_ISSUE(s, st)                                                                   \
  do {                                                                                            \
    const int piece_ = nx_piece, x0_ = piece_ * g.cw, y_ = nx_y;                                  \
    const uint32_t img_ = (uint32_t)nx_img;                                                       \
    if (++nx_piece == g.nchunks) {                                                                \
      nx_piece = 0;                                                                               \
      if (++nx_y == g.ho) { nx_y = 0; ++nx_img; }                                                 \
    }                                                                                             \
    const int top_ = S * y_ - g.pad;                                                              \
    if (top_ >= 0 && top_ + KS <= g.hs) {                                                         \
      float *sa_ = smem + (st) * stage + wave * 64;                                               \
      const uint32_t ga_ =                                                                        \
          (uint32_t)(((size_t)img_ * g.dout_img_stride + (size_t)m0 * ho2 + y_ * g.ho + x0_) * 4); \
      float *sb_ = sa_ + g.a_floats;                                                              \
      const uint32_t gb_ = (uint32_t)(((size_t)img_ * g.src_img_stride + (size_t)ch0 * hs2 +      \
                                       (size_t)top_ * g.hs + (size_t)S * x0_) * 4);               \
      /* counts and strides read afresh: kept across the loop they (and every multiple the loads use) would be */ \
      /* scalar registers spilled to lanes and read back with a vector instruction apiece            */ \
      int nal_ = g.nal, nbl_ = g.nbl, nth_ = nthreads;                                            \
      asm volatile("" : "+s"(nal_), "+s"(nbl_), "+s"(nth_));                                      \
      if (g.nchunks == 1 || (piece_ > 0 && piece_ < g.nchunks - 1)) {                             \
        _Pragma("unroll") for (int k = 0; k < NAL; ++k) {                                         \
          if (__builtin_expect(k < nal_, 1)) lds_dma4(a_rsrc, aoff[k], ga_, sa_ + k * nth_);     \
        }                                                                                         \
        _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                         \
          if (__builtin_expect(k < nbl_, 1)) lds_dma4(b_rsrc, boff[k], gb_, sb_ + k * nth_);     \
        }                                                                                         \
      } else {                                                                                    \
        /* first or last piece of a row: the words it lacks get the top offset bit (out of range) */ \
        const uint32_t na_ = piece_ == g.nchunks - 1 ? ~a_last : 0u;                              \
        const uint32_t nb_ = (piece_ == 0 ? ~b_first : 0u) | (piece_ == g.nchunks - 1 ? ~b_last : 0u); \
        _Pragma("unroll") for (int k = 0; k < NAL; ++k) {                                         \
          if (__builtin_expect(k < nal_, 1))                                                      \
            lds_dma4(a_rsrc, aoff[k] | (((na_ >> k) & 1u) << 31), ga_, sa_ + k * nth_);           \
        }                                                                                         \
        _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                         \
          if (__builtin_expect(k < nbl_, 1))                                                      \
            lds_dma4(b_rsrc, boff[k] | (((nb_ >> k) & 1u) << 31), gb_, sb_ + k * nth_);           \
        }                                                                                         \
      }                                                                                           \
      break;                                                                                      \
    }                                                                                             \
    const uint32_t ma_ = piece_ == g.nchunks - 1 ? a_last : ~0u;                                  \
    const uint32_t mb_ = (piece_ == 0 ? b_first : ~0u) & (piece_ == g.nchunks - 1 ? b_last : ~0u); \
    float *sa_ = smem + (st) * stage + wave * 64;                                                 \
    const uint32_t ga_ =                                                                          \
        (uint32_t)(((size_t)img_ * g.dout_img_stride + (size_t)m0 * ho2 + y_ * g.ho + x0_) * 4);  \
    _Pragma("unroll") for (int k = 0; k < NAL; ++k) {                                             \
      if (k < g.nal) lds_dma4(a_rsrc, ((ma_ >> k) & 1u) ? aoff[k] : kOutOfRange, ga_, sa_ + k * nthreads); \
    }                                                                                             \
    float *sb_ = sa_ + g.a_floats;                                                                \
    const uint32_t gb_ =                                                                          \
        (uint32_t)(((size_t)img_ * g.src_img_stride + (size_t)ch0 * hs2 + (size_t)S * x0_) * 4);  \
    /* the first patch row may lie above the image: that (negative) term goes into the lane     */ \
    /* offset, whose sum is non-negative for every lane that passes the row test                */ \
    const uint32_t row0_ = (uint32_t)(top_ * g.hs * 4);                                           \
    _Pragma("unroll") for (int k = 0; k < NBL; ++k) {                                             \
      const int srow_ = top_ + (int)((brow[k / 5] >> (6 * (k % 5))) & 63u);                       \
      const bool ok_ = (int)boff[k] >= 0 && ((mb_ >> k) & 1u) && (unsigned)srow_ < (unsigned)g.hs; \
      if (k < g.nbl) lds_dma4(b_rsrc, ok_ ? boff[k] + row0_ : kOutOfRange, gb_, sb_ + k * nthreads); \
    }                                                                                             \
  } while (0)

  // ---- fragment bases ----------------------------------------------------------------------
  const int abase = (wmi * 32 + r) * g.ast + h;
  int bbase[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = min(n0 + (wni * TB + b) * 32 + r, g.ncols - 1);
    const int c = col / KK, j = col - c * KK, u = j / KS, v = j - u * KS;
    bbase[b] = g.a_floats + (c - ch0) * g.pch + u * g.pws + v + S * h;
  }

  v16f acc[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
  float bsum = 0.0f;  // lane (r, h) adds up dout[map r][every image][every row][x = h (mod 2)]
  const bool want_bias = g.out_bias && tn == 0 && wni == 0;  // wavefront-uniform

  if (s_beg < s_end) {
    CCT_SWGRAD_ISSUE(s_beg, 0);
    lds_dma_wait();
  }
  __syncthreads();

  for (int s = s_beg; s < s_end; ++s) {
    const int cur = (s - s_beg) & 1;
    if (s + 1 < s_end) CCT_SWGRAD_ISSUE(s + 1, cur ^ 1);
    // LDS addresses of this lane's fragments at pixel 0 of the step, as registers of their own that advance once per
    // trip of the pixel loop (left to itself the compiler re-adds the stage to every one of them every trip:
    // vector ALU instructions take MFMA issue slots)
    typedef __attribute__((address_space(3))) const float lds_cfloat;
    lds_cfloat *ia = (lds_cfloat *)smem + (cur * stage + abase), *ib[TB];
    asm volatile("" : "+v"(ia));
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      ib[b] = (lds_cfloat *)smem + (cur * stage + bbase[b]);
      asm volatile("" : "+v"(ib[b]));
    }
    // fragment buffers; reads past ho stay inside the stage and meet zero dout words
    float fa[2], fb[2][TB];
#define CCT_SWGRAD_FRAGS(buf, x)                                                                  \
  do {                                                                                            \
    fa[buf] = ia[(x)];                                                                            \
    _Pragma("unroll") for (int b = 0; b < TB; ++b) fb[buf][b] = ib[b][S * (x)];                   \
  } while (0)
#define CCT_SWGRAD_MFMA(buf)                                                                      \
  do {                                                                                            \
    _Pragma("unroll") for (int b = 0; b < TB; ++b)                                                \
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf], fb[buf][b], acc[b], 0, 0, 0);      \
  } while (0)
// issue order of one pixel pair: the LDS reads of the next pair go out between this pair's MFMAs
#define CCT_SWGRAD_ORDER()                                                                        \
  do {                                                                                            \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                            \
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                                            \
    _Pragma("unroll") for (int k2 = 1; k2 < TB; ++k2) {                                           \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                          \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                          \
    }                                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                            \
  } while (0)
// four pixels from offset x of the address registers; the wavefronts that own a part of the bias gradient (few)
// add up their dout fragments, behind a scalar branch
#define CCT_SWGRAD_QUAD(x)                                                                        \
  do {                                                                                            \
    CCT_SWGRAD_FRAGS(1, (x) + 2);                                                                 \
    CCT_SWGRAD_MFMA(0);                                                                           \
    CCT_SWGRAD_ORDER();                                                                           \
    if (__builtin_expect(bias_flag != 0, 0)) bsum += fa[0] + fa[1];                               \
    CCT_SWGRAD_FRAGS(0, (x) + 4);                                                                 \
    CCT_SWGRAD_MFMA(1);                                                                           \
    CCT_SWGRAD_ORDER();                                                                           \
  } while (0)
    {
      int bias_flag = __builtin_amdgcn_readfirstlane(want_bias ? 1 : 0);
      asm volatile("" : "+s"(bias_flag));  // a scalar test every time, not a lane mask and a select
      CCT_SWGRAD_FRAGS(0, 0);
      int qd = 0;
      for (; qd + 2 <= g.nq2; qd += 2) {
        CCT_SWGRAD_QUAD(0);
        CCT_SWGRAD_QUAD(4);
        ia += 8;
        asm volatile("" : "+v"(ia));
#pragma unroll
        for (int b = 0; b < TB; ++b) {
          ib[b] += 8 * S;
          asm volatile("" : "+v"(ib[b]));
        }
      }
      if (qd < g.nq2) CCT_SWGRAD_QUAD(0);
    }
#undef CCT_SWGRAD_QUAD
#undef CCT_SWGRAD_FRAGS
#undef CCT_SWGRAD_MFMA
#undef CCT_SWGRAD_ORDER
    lds_dma_wait();
    __syncthreads();
  }
#undef CCT_SWGRAD_ISSUE

  if (want_bias) {
    const float both = bsum + __shfl_xor(bsum, 32);
    const int row = m0 + wmi * 32 + r;
    if (h == 0 && row < g.o) g.out_bias[(size_t)z * g.o + row] = both;
  }
  float *out = g.out + (size_t)z * g.o * g.ncols;
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = n0 + (wni * TB + b) * 32 + r;
    if (col >= g.ncols) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wmi * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < g.o) out[(size_t)row * g.ncols + col] = acc[b][v];
    }
  }
}

// The same computation for layers without padding whose output-row length and load counts are
// known at compile time (conv1 of AlexNet / CaffeNet).  Vector-ALU instructions do not overlap with
// the MFMAs of the same SIMD, so this variant issues next to none inside a step: the step is one
// straight line of code, every fragment read is base register + immediate offset, the step-dependent
// part of every global address sits in the scalar offset of the buffer load (no padding: the rows
// under an output row are always inside the image), the next step's loads are spread between the
// MFMAs of this one (unconditionally: the last step of a range re-fetches itself into the idle
// stage), and the bias gradient costs no additions at all: the first unused column of the padded
// column range reads a row of ones, so its accumulator column IS the sum of dout.
constexpr int kSWgradOnes = 256;  // floats of the row of ones (>= S * pixels of a padded output row)

template <int KS, int S, int TB, int NQ2, int NAL, int NBL>
__global__ __launch_bounds__(768) void conv_strided_wgrad_spec_kernel(const StridedWgradArgs g) {
  constexpr int KK = KS * KS;
  constexpr int NP = 2 * NQ2;          // pixel pairs per step
  constexpr int NSLOT = NAL + NBL;     // global -> LDS loads per lane per step
  constexpr int NQI = (NP * 5 + 7) / 8;  // pairs that carry a slice of the loads (the last ones leave time to land)
  static_assert(S * (2 * NP + 1) < kSWgradOnes, "row of ones too short");
  extern __shared__ __attribute__((aligned(16))) float smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nthreads = blockDim.x;
  const int r = lane & 31, h = lane >> 5;
  const int wni = (int)fdiv((uint32_t)wave, g.div_wm), wmi = wave - wni * g.wm;
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t z = flat / g.ntiles, id = flat - z * g.ntiles;
  const uint32_t tm = id / g.tiles_n, tn = id - tm * g.tiles_n;
  const int bm = 32 * g.wm;
  const int m0 = tm * bm, n0 = tn * (32 * TB * g.wn), ch0 = n0 / KK;
  const int s_beg = z * g.steps_per_split, s_end = min(g.steps_total, s_beg + g.steps_per_split);
  const int ho2 = g.ho * g.ho, hs2 = g.hs * g.hs;
  const int stage = g.a_floats + g.b_floats;
  float *const ones = smem + 2 * stage;
  for (int i = tid; i < kSWgradOnes; i += nthreads) ones[i] = 1.0f;

  uint32_t aoff[NAL];  // byte offset from (image, map m0, row y); kOutOfRange = a zero word
#pragma unroll
  for (int k = 0; k < NAL; ++k) {
    const uint32_t e = (uint32_t)(k * nthreads + tid);
    const uint32_t m = fdiv(e, g.div_ast), i = e - m * g.ast;
    const bool ok = m < (uint32_t)bm && m0 + (int)m < g.o && i < (uint32_t)g.ho;
    aoff[k] = ok ? (m * ho2 + i) * 4u : kOutOfRange;
  }
  uint32_t boff[NBL];  // byte offset from (image, channel ch0, row S*y); kOutOfRange = a zero word
#pragma unroll
  for (int k = 0; k < NBL; ++k) {
    const uint32_t e = (uint32_t)(k * nthreads + tid);
    const uint32_t ch = fdiv(e, g.div_pch), rem = e - ch * g.pch;
    const uint32_t prow = fdiv(rem, g.div_pws), pcol = rem - prow * g.pws;
    const bool ok = ch < (uint32_t)g.nch && prow < (uint32_t)KS && ch0 + (int)ch < g.d && pcol < (uint32_t)g.hs;
    boff[k] = ok ? (ch * hs2 + prow * g.hs + pcol) * 4u : kOutOfRange;
  }
  const rsrc_t a_rsrc = make_rsrc(g.dout), b_rsrc = make_rsrc(g.src);

  const int abase = (wmi * 32 + r) * g.ast + h;
  int bbase[TB];
  bool bias_col[TB];  // this lane's column of block b is the column of ones
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col_raw = n0 + (wni * TB + b) * 32 + r;
    const int col = min(col_raw, g.ncols - 1);
    const int c = col / KK, j = col - c * KK, u = j / KS, v = j - u * KS;
    bbase[b] = g.a_floats + (c - ch0) * g.pch + u * g.pws + v + S * h;
    bias_col[b] = col_raw == g.ncols;
  }

  v16f acc[TB];
#pragma unroll
  for (int b = 0; b < TB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;

// scalars of step s: the scalar offsets of its slab and patch loads
#define CCT_SWSPEC_STEP(s)                                                                        \
  const uint32_t img_ = fdiv((uint32_t)(s), g.div_ho);                                            \
  const int y_ = (s) - (int)img_ * g.ho;                                                          \
  const uint32_t ga_ = (uint32_t)(((size_t)img_ * g.dout_img_stride + (size_t)m0 * ho2 + y_ * g.ho) * 4); \
  const uint32_t gb_ = (uint32_t)(((size_t)img_ * g.src_img_stride + (size_t)ch0 * hs2 + (size_t)S * y_ * g.hs) * 4)
#define CCT_SWSPEC_SLOT(k, st)                                                                    \
  do {                                                                                            \
    if ((k) < NAL)                                                                                \
      lds_dma4(a_rsrc, aoff[(k) < NAL ? (k) : 0], ga_, smem + (st) * stage + wave * 64 + (k) * nthreads); \
    else                                                                                          \
      lds_dma4(b_rsrc, boff[(k) >= NAL ? (k) - NAL : 0], gb_,                                     \
               smem + (st) * stage + g.a_floats + wave * 64 + ((k) - NAL) * nthreads);            \
  } while (0)

  if (s_beg < s_end) {
    CCT_SWSPEC_STEP(s_beg);
#pragma unroll
    for (int k = 0; k < NSLOT; ++k) CCT_SWSPEC_SLOT(k, 0);
    lds_dma_wait();
  }
  __syncthreads();

  for (int s = s_beg; s < s_end; ++s) {
    const int cur = (s - s_beg) & 1, nxt = cur ^ 1;
    CCT_SWSPEC_STEP(min(s + 1, s_end - 1));
    const float *sa = smem + cur * stage + abase;
    const float *sb[TB];
#pragma unroll
    for (int b = 0; b < TB; ++b) sb[b] = bias_col[b] ? ones : smem + cur * stage + bbase[b];
    float fa[2], fb[2][TB];
#define CCT_SWSPEC_FRAGS(buf, x)                                                                  \
  do {                                                                                            \
    fa[buf] = sa[(x)];                                                                            \
    _Pragma("unroll") for (int b = 0; b < TB; ++b) fb[buf][b] = sb[b][S * (x)];                   \
  } while (0)
    CCT_SWSPEC_FRAGS(0, 0);
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int cb = q & 1, nb = cb ^ 1;
      if (q + 1 < NP) CCT_SWSPEC_FRAGS(nb, 2 * q + 2);
#pragma unroll
      for (int b = 0; b < TB; ++b)
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb], fb[cb][b], acc[b], 0, 0, 0);
      // this pair's share of the next step's loads
      const int qi = q < NQI ? q : NQI, qj = q + 1 < NQI ? q + 1 : NQI;
      const int k_lo = qi * NSLOT / NQI, k_hi = qj * NSLOT / NQI;
#pragma unroll
      for (int k = 0; k < NSLOT; ++k)
        if (k >= k_lo && k < k_hi) CCT_SWSPEC_SLOT(k, nxt);
      // issue order: an LDS read of the next pair after every MFMA (two after the first), then the global loads
      {
        const int nr = q + 1 < NP ? TB + 1 : 0;
        int left_r = nr, left_v = k_hi - k_lo;
#pragma unroll
        for (int k2 = 0; k2 < TB; ++k2) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          const int take_r = left_r > 0 ? (k2 == 0 && left_r > 1 ? 2 : 1) : 0;
          if (take_r == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          else if (take_r == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          left_r -= take_r;
          if (left_v > 0) {
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            --left_v;
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#undef CCT_SWSPEC_FRAGS
    lds_dma_wait();
    __syncthreads();
  }
#undef CCT_SWSPEC_STEP
#undef CCT_SWSPEC_SLOT

  float *out = g.out + (size_t)z * g.o * g.ncols;
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int col = n0 + (wni * TB + b) * 32 + r;
    if (col > g.ncols || (col == g.ncols && !g.out_bias)) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + wmi * 32 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row >= g.o) continue;
      if (col == g.ncols) g.out_bias[(size_t)z * g.o + row] = acc[b][v];  // the column of ones: sum of dout
      else out[(size_t)row * g.ncols + col] = acc[b][v];
    }
  }
}

struct StridedWgradPlan {
  int tb, wm, wn, nch, ast, a_floats, b_floats, nal, nbl, pws, pch, nq2;
  int cw, nchunks;  // pieces an output row is taken in: nchunks of cw pixels (ho, 1 where a row fits a step)
  bool spec;  // a compile-time specialised instance exists for this shape
  size_t lds;
};

static bool strided_kernel_size(int ks, int stride) {
  return (ks == 11 && stride == 4) || (ks == 7 && stride == 2) || (ks == 5 && stride == 2) || (ks == 3 && stride == 2);
}
// the weight-gradient kernel also has stride-1 instances (3 x 3 and 5 x 5): the stride-1 kernels of their own
// file stage image PAIRS and stop at padded rows of 32 floats, this one takes rows as long as its patch holds
static bool strided_wgrad_kernel_size(int ks, int stride) {
  return strided_kernel_size(ks, stride) || (stride == 1 && (ks == 3 || ks == 5 || ks == 7));
}

// Chooses the workgroup shape for a geometry; false when the strided weight-gradient kernel does not cover it.
static bool strided_wgrad_plan(int batch, int d, int n, int ks, int stride, int pad, int o, StridedWgradPlan *pl) {
  if (!strided_wgrad_kernel_size(ks, stride)) return false;
  if (batch <= 0 || d <= 0 || o <= 0 || pad < 0 || pad >= ks || n + 2 * pad < ks) return false;
  const int hp = n + 2 * pad, ho = (hp - ks) / stride + 1, kk = ks * ks;
  if ((double)batch * d * n * n >= 536870912.0 || (double)batch * o * ho * ho >= 536870912.0 ||
      (double)o * d * kk >= 536870912.0)
    return false;  // 32-bit byte offsets
  const int ncols = d * kk, cb = (ncols + 31) / 32, mb = (o + 31) / 32;
  double best_cost = -1;
  // An output row is taken whole or in up to 64 balanced pieces (the last piece wide enough that only it can reach
  // past the image's right edge): as few as the slab and patch loads of a step allow for the tile, since every step
  // costs a barrier and a pipeline refill -- about what 13 more pixels would.
  const int forced = tuning().strided_wgrad;
  for (int nchunks = 1; nchunks <= 64; ++nchunks) {
  if (forced && nchunks != forced / 1000) continue;
  const int cw = (ho + nchunks - 1) / nchunks, last_w = ho - (nchunks - 1) * cw;
  if (nchunks > 1 && (last_w < 1 || last_w * stride < ks || cw < ks)) continue;
  const int nq2 = (cw + 3) / 4, ast = 4 * nq2 + 1;
  const int tw = stride * (cw - 1) + ks;                      // source columns a piece of an output row touches
  const int pws = tw + (((ks - tw) % 32) + 32) % 32;          // >= tw, == ks (mod 32)
  const int raw = ks * pws, pch = raw + (((kk - raw) % 32) + 32) % 32;  // >= raw, == ks*ks (mod 32)
  // candidates: column blocks per wavefront x column groups x row blocks; cost = MFMAs issued per step
  for (int tb = 3; tb >= 1; --tb)
    for (int wn = 4; wn >= 1; --wn)
      for (int wm = 4; wm >= 1; --wm) {
        const int w = wm * wn;
        if (w > 12) continue;
        if (forced && forced % 1000 != tb * 100 + wn * 10 + wm) continue;
        if (wm > mb || (wn - 1) * tb >= cb) continue;  // wavefronts with nothing to do
        const int nth = 64 * w;
        const int tiles_n = (cb + tb * wn - 1) / (tb * wn), tiles_m = (mb + wm - 1) / wm;
        int nch = (32 * tb * wn - 1) / kk + 2;
        if (nch > d) nch = d;
        // last word a fragment load can touch: the step's final prefetch reads pixel 4*nq2 + 1
        const int b_need = (nch - 1) * pch + (ks - 1) * pws + (ks - 1) + stride * (4 * nq2 + 1) + 1;
        const int b_floats = ((b_need > nch * pch ? b_need : nch * pch) + nth - 1) / nth * nth;
        const int a_floats = (32 * wm * ast + 2 + nth - 1) / nth * nth;
        const int nal = a_floats / nth, nbl = b_floats / nth;
        if (nal > kSWgradSlabLoads || nbl > kSWgradPatchLoads) continue;
        const size_t lds = (size_t)2 * (a_floats + b_floats) * sizeof(float);
        if (lds > 160 * 1024) continue;
        // Padded MFMA work, step overhead included, over the rate of the tile relative to one column block per
        // wavefront: with three blocks a wavefront reads four LDS fragments per three MFMAs instead of two per
        // one (measured 1.26 and 1.33 for two and three blocks on 96 -> 96 maps of 5 x 5 at 96 x 96 and on
        // 128 -> 128 maps of 3 x 3 at 112 x 112); twelve wavefronts hide a step's barrier better than eight or four
        // (1.0 : 0.92 : 0.9 there); a wavefront count that loads the four SIMDs unevenly loses more than its padding
        // saves (six wavefronts against four on 64 -> 64 maps of 7 x 7, stride 2: 0.24 against 0.17 ms).
        static const double tb_rate[4] = {0, 1.0, 1.26, 1.33};
        double cost = (double)tiles_n * tb * wn * tiles_m * wm * nchunks * (4 * nq2 + 13) / tb_rate[tb];
        cost /= w >= 12 ? 1.0 : w >= 8 ? 0.92 : w >= 4 ? 0.9 : 0.85;
        if (w % 4) cost *= 1.15;
        if (best_cost < 0 || cost < best_cost) {
          best_cost = cost;
          pl->tb = tb; pl->wm = wm; pl->wn = wn; pl->nch = nch; pl->ast = ast; pl->a_floats = a_floats;
          pl->b_floats = b_floats; pl->nal = nal; pl->nbl = nbl; pl->pws = pws; pl->pch = pch; pl->nq2 = nq2;
          pl->cw = cw; pl->nchunks = nchunks;
          pl->lds = lds;
        }
      }
  }
  if (best_cost < 0) return false;
  // conv1 of AlexNet / CaffeNet: 11 x 11, stride 4, no padding, 53..56 pixels per output row, a spare column
  pl->spec = ks == 11 && stride == 4 && pad == 0 && pl->tb == 3 && pl->nq2 == 14 && pl->nal == 8 && pl->nbl == 11 &&
             pl->nchunks == 1 && ncols % 32 != 0 && !tuning().direct_nospec;
  if (pl->spec) pl->lds += kSWgradOnes * sizeof(float);
  return pl->lds <= 160 * 1024;
}

template <int KS, int S>
static int strided_wgrad_launch(const StridedWgradArgs &g, const StridedWgradPlan &pl, hipStream_t st) {
  dim3 grid(g.nblocks), block(64 * pl.wm * pl.wn);
#define CCT_SWGRAD_CASE(TB)                                                                       \
  if (pl.tb == TB) {                                                                              \
    auto kern = conv_strided_wgrad_kernel<KS, S, TB>;                                             \
    static LdsGrant grant;                                                                        \
    if (int rc = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc;                 \
    hipLaunchKernelGGL(kern, grid, block, pl.lds, st, g);                                         \
    CCT_LAUNCH_CHECK();                                                                           \
    note_kernel("conv_strided_wgrad_kernel<%d,%d,%d> waves=%dx%d pieces=%d", KS, S, TB, pl.wm, pl.wn, pl.nchunks); \
    return 0;                                                                                     \
  }
  CCT_SWGRAD_CASE(1) CCT_SWGRAD_CASE(2) CCT_SWGRAD_CASE(3)
#undef CCT_SWGRAD_CASE
  return set_error(CCT_HIP_EINVAL, "conv_strided wgrad: no kernel instance for %d column blocks", pl.tb);
}

bool conv_strided_wgrad_covers(int batch, int d, int n, int ks, int stride, int pad, int o) {
  StridedWgradPlan pl;
  return strided_wgrad_plan(batch, d, n, ks, stride, pad, o, &pl);
}

int conv_strided_wgrad(float *dw, float *db, const float *dout, const float *src, int batch, int d, int n, int ks,
                       int stride, int pad, int o, size_t src_img_stride, size_t dout_img_stride) {
  StridedWgradPlan pl;
  CCT_REQUIRE(strided_wgrad_plan(batch, d, n, ks, stride, pad, o, &pl),
              "conv_strided wgrad: geometry not covered (k=%d stride=%d pad=%d size=%d)", ks, stride, pad, n);
  StridedWgradArgs g;
  g.dout = dout; g.src = src;
  g.batch = batch; g.o = o; g.d = d; g.hs = n; g.pad = pad;
  g.ho = (n + 2 * pad - ks) / stride + 1;
  g.ncols = d * ks * ks;
  g.wm = pl.wm; g.wn = pl.wn; g.nch = pl.nch; g.ast = pl.ast; g.a_floats = pl.a_floats; g.b_floats = pl.b_floats;
  g.nal = pl.nal; g.nbl = pl.nbl; g.pws = pl.pws; g.pch = pl.pch; g.nq2 = pl.nq2;
  g.cw = pl.cw; g.nchunks = pl.nchunks;
  g.steps_total = batch * g.ho * pl.nchunks;
  {
    const size_t dense_src = (size_t)d * n * n, dense_dout = (size_t)o * g.ho * g.ho;
    if (!src_img_stride) src_img_stride = dense_src;
    if (!dout_img_stride) dout_img_stride = dense_dout;
    CCT_REQUIRE(src_img_stride >= dense_src && dout_img_stride >= dense_dout,
                "conv_strided wgrad: image stride smaller than an image");
    CCT_REQUIRE((double)batch * src_img_stride < 536870912.0 && (double)batch * dout_img_stride < 536870912.0,
                "conv_strided wgrad: strided tensor too large for 32-bit byte offsets");
    g.src_img_stride = (uint32_t)src_img_stride;
    g.dout_img_stride = (uint32_t)dout_img_stride;
  }
  g.tiles_m = (uint32_t)((o + 32 * pl.wm - 1) / (32 * pl.wm));
  g.tiles_n = (uint32_t)((g.ncols + 32 * pl.tb * pl.wn - 1) / (32 * pl.tb * pl.wn));
  g.ntiles = g.tiles_m * g.tiles_n;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  // workgroups resident per compute unit: LDS, and three wavefronts per SIMD (the register budget of the kernel)
  int per_cu = (int)((160 * 1024) / pl.lds);
  if (per_cu > 12 / (pl.wm * pl.wn)) per_cu = 12 / (pl.wm * pl.wn);
  if (per_cu < 1) per_cu = 1;
  int splits = (int)((long)per_cu * cus / g.ntiles);
  if (splits < 1) splits = 1;
  if (splits > g.steps_total) splits = g.steps_total;
  g.steps_per_split = (g.steps_total + splits - 1) / splits;
  splits = (g.steps_total + g.steps_per_split - 1) / g.steps_per_split;
  g.nblocks = g.ntiles * (uint32_t)splits;
  g.div_ho = make_fastdiv((uint32_t)g.ho);
  g.div_ast = make_fastdiv((uint32_t)g.ast);
  g.div_pch = make_fastdiv((uint32_t)g.pch);
  g.div_pws = make_fastdiv((uint32_t)g.pws);
  g.div_wm = make_fastdiv((uint32_t)g.wm);
  g.div_nchunks = make_fastdiv((uint32_t)g.nchunks);
  const size_t n_out = (size_t)o * g.ncols;
  if (splits > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)splits * (n_out + (db ? o : 0)) * sizeof(float), &ws);
    if (rc) return rc;
    g.out = (float *)ws;
    g.out_bias = db ? g.out + (size_t)splits * n_out : nullptr;
  } else {
    g.out = dw;
    g.out_bias = db;
  }
  hipStream_t st = ctx().stream;
  int rc;
  if (pl.spec) {
    auto kern = conv_strided_wgrad_spec_kernel<11, 4, 3, 14, 8, 11>;
    static LdsGrant grant;
    if (int rc2 = grant_dynamic_lds((const void *)kern, pl.lds, grant)) return rc2;
    hipLaunchKernelGGL(kern, dim3(g.nblocks), dim3(64 * pl.wm * pl.wn), pl.lds, st, g);
    CCT_LAUNCH_CHECK();
    note_kernel("conv_strided_wgrad_spec_kernel<11,4,3,14,8,11> waves=%dx%d", pl.wm, pl.wn);
    rc = 0;
  } else if (ks == 11) rc = strided_wgrad_launch<11, 4>(g, pl, st);
  else if (ks == 7) rc = stride == 2 ? strided_wgrad_launch<7, 2>(g, pl, st) : strided_wgrad_launch<7, 1>(g, pl, st);
  else if (ks == 5) rc = stride == 2 ? strided_wgrad_launch<5, 2>(g, pl, st) : strided_wgrad_launch<5, 1>(g, pl, st);
  else rc = stride == 2 ? strided_wgrad_launch<3, 2>(g, pl, st) : strided_wgrad_launch<3, 1>(g, pl, st);
  if (rc) return rc;
  if (splits > 1)
    return reduce_partial_sums(dw, g.out, (uint32_t)n_out, db, g.out_bias, db ? (uint32_t)o : 0u, splits, st);
  return 0;
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_conv_strided_supported(int batch, int depth, int n, int k, int stride, int padding,
                                              int num_outputs) {
  StridedPlan pl;
  StridedWgradPlan wpl;
  return strided_plan(batch, depth, n, k, stride, padding, num_outputs, &pl) &&
                 strided_wgrad_plan(batch, depth, n, k, stride, padding, num_outputs, &wpl)
             ? 1
             : 0;
}

extern "C" size_t cct_hip_conv_strided_slab_floats(int num_outputs, int depth, int k, int stride, int padding) {
  StridedPlan pl;
  // the slab layout depends on the kernel size, the map count and on whether the layer pads
  if (!strided_plan(1, depth, 4 * k, k, stride, padding ? 1 : 0, num_outputs, &pl)) return 0;
  return padding ? (size_t)depth * pl.ksp * pl.mpad * pl.ast : (size_t)depth * pl.nst * pl.mpad * pl.ast_step;
}

extern "C" int cct_hip_conv_strided_slabs(float *slabs, const float *model, int num_outputs, int depth, int k,
                                          int stride, int padding) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(slabs && model, "conv_strided_slabs: null argument");
  StridedPlan pl;
  CCT_REQUIRE(strided_plan(1, depth, 4 * k, k, stride, padding ? 1 : 0, num_outputs, &pl),
              "conv_strided_slabs: kernel size %d with stride %d is not covered", k, stride);
  if (padding == 0) {
    const size_t total = (size_t)depth * pl.nst * pl.mpad * pl.ast_step;
    CCT_REQUIRE(total < (1ull << 31), "conv_strided_slabs: model too large");
    hipLaunchKernelGGL(conv_strided_step_slab_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx().stream,
                       slabs, model, depth, num_outputs, pl.mpad, k, pl.nst, pl.ast_step, (uint32_t)total,
                       make_fastdiv(pl.ast_step), make_fastdiv(pl.mpad), make_fastdiv(pl.nst), make_fastdiv(k));
    CCT_LAUNCH_CHECK();
    return 0;
  }
  const size_t total = (size_t)depth * pl.ksp * pl.mpad * pl.ast;
  CCT_REQUIRE(total < (1ull << 31), "conv_strided_slabs: model too large");
  hipLaunchKernelGGL(conv_strided_slab_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx().stream, slabs,
                     model, depth, num_outputs, pl.mpad, k, pl.ksp, pl.ast, (uint32_t)total, make_fastdiv(pl.ast),
                     make_fastdiv(pl.mpad), make_fastdiv(pl.ksp));
  CCT_LAUNCH_CHECK();
  return 0;
}

extern "C" int cct_hip_conv_strided_forward(float *output, const float *input, const float *slabs, const float *bias,
                                            int batch, int depth, int n, int k, int stride, int padding,
                                            int num_outputs, int relu) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(output && input && slabs, "conv_strided_forward: null argument");
  StridedPlan pl;
  CCT_REQUIRE(strided_plan(batch, depth, n, k, stride, padding, num_outputs, &pl),
              "conv_strided_forward: geometry not covered (k=%d stride=%d pad=%d size=%d)", k, stride, padding, n);
  CCT_REQUIRE((uintptr_t)slabs % 16 == 0, "conv_strided_forward: slab buffer must be 16-byte aligned");
  StridedArgs g;
  g.wt = slabs; g.src = input; g.dst = output; g.bias = bias; g.relu = relu;
  g.batch = batch; g.kc = depth; g.mtot = num_outputs; g.mpad = pl.mpad; g.hs = n; g.pad = padding;
  g.hp = n + 2 * padding;
  g.ho = (g.hp - k) / stride + 1;
  g.xw = pl.xw; g.rs = pl.rs; g.pr = pl.pr;
  g.ptot = (uint32_t)((long)batch * g.ho * g.ho);
  g.tiles_m = (uint32_t)(pl.mpad / (32 * pl.tmb));
  g.ntiles = g.tiles_m * ((g.ptot + 127) / 128);
  g.div_ho = make_fastdiv((uint32_t)g.ho);
  g.div_ho2 = make_fastdiv((uint32_t)(g.ho * g.ho));
  g.div_hp = make_fastdiv((uint32_t)g.hp);
  g.div_rs = make_fastdiv((uint32_t)g.rs);
  g.div_xw = make_fastdiv((uint32_t)g.xw);
  hipStream_t st = ctx().stream;
  if (k == 11 && stride == 4) return strided_launch<11, 4>(g, pl, st);
  if (k == 7 && stride == 2) return strided_launch<7, 2>(g, pl, st);
  if (k == 5 && stride == 2) return strided_launch<5, 2>(g, pl, st);
  return strided_launch<3, 2>(g, pl, st);
}

extern "C" int cct_hip_conv_strided_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                                     const float *input, int batch, int depth, int n, int k,
                                                     int stride, int padding, int num_outputs) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(model_grad && output_grad && input, "conv_strided_backward_weights: null argument");
  CCT_REQUIRE(stride > 1, "conv_strided_backward_weights: stride-1 layers go through cct_hip_conv_direct_backward_weights");
  return conv_strided_wgrad(model_grad, bias_grad, output_grad, input, batch, depth, n, k, stride, padding,
                            num_outputs, 0, 0);
}
