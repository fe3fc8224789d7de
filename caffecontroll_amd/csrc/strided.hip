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
  if ((double)batch * d * n * n >= 1073741824.0 || (double)batch * o * ho * ho >= 1073741824.0) return false;
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

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_conv_strided_supported(int batch, int depth, int n, int k, int stride, int padding,
                                              int num_outputs) {
  StridedPlan pl;
  return strided_plan(batch, depth, n, k, stride, padding, num_outputs, &pl) ? 1 : 0;
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
