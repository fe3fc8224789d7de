// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32), cblas_sgemm contract.
//
//   C[M x N] = alpha * op(A)[M x K] * op(B)[K x N] + beta * C        (row-major view)
//
// Structure of one workgroup (256 lanes = 4 wavefronts):
//   * macro tile BM x BN of C, K consumed in steps of BK through LDS, two LDS stages
//     (global loads for step t+1 are issued before the MFMAs of step t and parked in registers,
//     then written to the other stage; one barrier per step);
//   * each wavefront owns a WM x WN sub-tile made of 32x32 MFMA accumulators;
//   * LDS layout follows the operand's contiguous direction so that global reads and LDS writes
//     are 16-byte vectors in both cases:
//       K-contiguous operand   -> [row][BK + 4]   fragments fetched as one ds_read_b128 per 4 MFMAs
//       row-contiguous operand -> [BK][rows + 8]  fragments fetched as conflict-free ds_read_b32
//     (the MFMA sums over k in any order, so both operands use the k-permutation
//      k = 8*kg + 4*half + i for MFMA i of group kg, half = lane/32);
//   * epilogues: plain alpha/beta; raw partial sums for split-K (reduced by a second kernel in a
//     fixed order, so results are run-to-run identical); forward-convolution epilogue that
//     writes [b][o][fmap] directly and adds the bias.
//
// Bound: fp32 MFMA rate (256 FLOP/clk/CU).  Algorithmic work 2*M*N*K FLOP per call.
#include <cstdlib>

#include "cct_common.h"
#include "colsum.h"
#include "mfma_common.h"

namespace cct {

// (v16f and f4 -- a native 4-float vector, which stays in registers where HIP's float4 struct can end
// up in scratch -- come from mfma_common.h)
// the same vector where only dword alignment may be assumed (global memory operands)
typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));

enum EpilogueMode { EPI_ALPHA_BETA = 0, EPI_SPLITK_PARTIAL = 1, EPI_CONV_FORWARD = 2 };

struct GemmArgs {
  const float *A;
  const float *B;
  float *C;
  int M, N, K;
  int lda, ldb, ldc;
  float alpha, beta;
  int kchunk;       // K range per grid.y slice (multiple of BK)
  float *ws;        // split-K partials [grid.y][M][N]
  int epi;
  int fmap;         // EPI_CONV_FORWARD: columns per image
  FastDiv div_fmap;
  const float *bias;
  int relu;         // clamp at zero after the bias (EPI_CONV_FORWARD; EPI_ALPHA_BETA with col_bias)
  const float *col_bias;  // EPI_ALPHA_BETA: added to every row of C (one value per column), or null
  int tiles_m, tiles_n;
  uint32_t ntiles;
  int a_vec, b_vec;  // operand allows aligned 16-byte global loads
  int splits;        // K slices; grid = ntiles * splits workgroups
  uint32_t nblocks;
  int nt_store;      // stream the output with non-temporal stores (large outputs that are not re-read)
  int dma;           // operands go global -> LDS without passing through registers (gemm_mainloop_dma)
  // A batch of products in one launch (1 x 1 convolution on [image][channel][pixel] tensors).  The grid's slice
  // index (what selects a K range otherwise) selects images; a slice covers the whole K.
  //   bmode 1: one product per image, image i with A + i*a_bstride, B + i*b_bstride, C + i*c_bstride;
  //   bmode 2: ONE product summed over the images, slice z = (image group, K range): it adds K range
  //            z % bksplit (kchunk wide) of images (z / bksplit)*bgroup .. +bgroup-1 (of nbatch) and stores like
  //            a K slice does (partial sums for the reduction when there are several slices).
  //   bmode 3: ONE product whose columns run over the pixels of ALL images (column n = image n / bplane, pixel
  //            n % bplane): B(k, n) sits at B + image*b_bstride + k*ldb + pixel, C is stored by the forward
  //            convolution's epilogue ([image][row][pixel]); no tile is padded per image.
  int bmode, nbatch, bgroup, bksplit;
  size_t a_bstride, b_bstride, c_bstride;  // floats
  uint32_t bplane;
  FastDiv div_bplane;
};

// Columns of a row-contiguous B operand numbered across images (GemmArgs::bmode 3); plane = 0: plain columns.
struct ImageCols {
  uint32_t plane;
  FastDiv div;
  size_t stride;  // floats between images
  __device__ __forceinline__ size_t offset(uint32_t n) const {  // float offset of column n within row k = 0
    const uint32_t img = fdiv(n, div);
    return (size_t)img * stride + (n - img * plane);
  }
};

__device__ __forceinline__ f4 ldg4(const float *__restrict__ base, int major, int minor,
                                       int major_lim, int minor_lim, int ld, int vec) {
  f4 v = f4{0.f, 0.f, 0.f, 0.f};
  if (major < major_lim) {
    const float *p = base + (size_t)major * ld + minor;
    if (vec && minor + 3 < minor_lim) {
      v = *reinterpret_cast<const f4u *>(p);
    } else {
      if (minor + 0 < minor_lim) v.x = p[0];
      if (minor + 1 < minor_lim) v.y = p[1];
      if (minor + 2 < minor_lim) v.z = p[2];
      if (minor + 3 < minor_lim) v.w = p[3];
    }
  }
  return v;
}

// the same for a row of B whose columns are numbered across images: every element has an address of its own
__device__ __forceinline__ f4 ldg4_cols(const float *__restrict__ base, int k, int col, int k_lim, int col_lim, int ld,
                                        const ImageCols &ic) {
  f4 v = f4{0.f, 0.f, 0.f, 0.f};
  if (k < k_lim) {
    const float *p = base + (size_t)k * ld;
    if (col + 0 < col_lim) v.x = p[ic.offset(col)];
    if (col + 1 < col_lim) v.y = p[ic.offset(col + 1)];
    if (col + 2 < col_lim) v.z = p[ic.offset(col + 2)];
    if (col + 3 < col_lim) v.w = p[ic.offset(col + 3)];
  }
  return v;
}

template <int BM_, int BN_, int BK_, int WGM_, int WGN_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
  static constexpr int THREADS = WGM * WGN * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int PK = 4;  // pad of K-contiguous LDS rows
  static constexpr int PR = 8;  // pad of row-contiguous LDS rows
  static_assert(BK % 8 == 0, "BK must hold whole k-groups");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 MFMA tiles");
  static_assert((BM * BK / 4) % 64 == 0 && (BN * BK / 4) % 64 == 0, "whole wavefronts load an operand tile");
};

template <class T, bool KC, int ROWS>
struct OperandLayout {
  // floats per LDS stage
  static constexpr int SIZE = KC ? ROWS * (T::BK + T::PK) : T::BK * (ROWS + T::PR);
  static constexpr int TOTAL = ROWS * T::BK / 4;                        // f4 per stage
  static constexpr int NV = (TOTAL + T::THREADS - 1) / T::THREADS;      // f4 per lane per stage
  // Slot i of a lane exists when its f4 index is inside the tile; only the last slot can be partial
  // (a 96-row tile loaded by 256 lanes: 1.5 f4 per lane), and then whole wavefronts are in or out.
  static __device__ __forceinline__ bool active(int i, int tid) {
    return (i + 1) * T::THREADS <= TOTAL || tid + i * T::THREADS < TOTAL;
  }
};

// global -> registers for one operand tile (rows x BK) starting at (row0, k0)
template <class T, bool KC, int ROWS>
__device__ __forceinline__ void load_tile(f4 *__restrict__ r,
                                          const float *__restrict__ g, int ld, int row0, int k0,
                                          int row_lim, int k_lim, int vec, int tid, const ImageCols *ic = nullptr) {
  using L = OperandLayout<T, KC, ROWS>;
  constexpr int NV = L::NV;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (!L::active(i, tid)) continue;
    const int f = tid + i * T::THREADS;
    if (KC) {
      const int row = f / (T::BK / 4), kq = f % (T::BK / 4);
      r[i] = ldg4(g, row0 + row, k0 + kq * 4, row_lim, k_lim, ld, vec);
    } else {
      const int kk = f / (ROWS / 4), rq = f % (ROWS / 4);
      if (ic && ic->plane) r[i] = ldg4_cols(g, k0 + kk, row0 + rq * 4, k_lim, row_lim, ld, *ic);
      else r[i] = ldg4(g, k0 + kk, row0 + rq * 4, k_lim, row_lim, ld, vec);
    }
  }
}

template <class T, bool KC, int ROWS>
__device__ __forceinline__ void store_tile(float *__restrict__ lds, const f4 *__restrict__ r,
                                           int tid) {
  using L = OperandLayout<T, KC, ROWS>;
  constexpr int NV = L::NV;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (!L::active(i, tid)) continue;
    const int f = tid + i * T::THREADS;
    if (KC) {
      const int row = f / (T::BK / 4), kq = f % (T::BK / 4);
      *reinterpret_cast<f4 *>(lds + row * (T::BK + T::PK) + kq * 4) = r[i];
    } else {
      const int kk = f / (ROWS / 4), rq = f % (ROWS / 4);
      *reinterpret_cast<f4 *>(lds + kk * (ROWS + T::PR) + rq * 4) = r[i];
    }
  }
}

// fragments of k-group kg for NT 32-row tiles starting at row0: component i of f[t] feeds MFMA i
// of the group
template <class T, bool KC, int ROWS, int NT>
__device__ __forceinline__ void load_frags(f4 (&f)[NT], const float *__restrict__ lds, int row0, int kg,
                                           int lane) {
  const int r = lane & 31, h = lane >> 5;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (KC) {
      f[t] = *reinterpret_cast<const f4 *>(lds + (row0 + t * 32 + r) * (T::BK + T::PK) + kg * 8 + h * 4);
    } else {
      const float *p = lds + (kg * 8 + h * 4) * (ROWS + T::PR) + row0 + t * 32 + r;
      f[t].x = p[0];
      f[t].y = p[ROWS + T::PR];
      f[t].z = p[2 * (ROWS + T::PR)];
      f[t].w = p[3 * (ROWS + T::PR)];
    }
  }
}

template <int I>
__device__ __forceinline__ float comp(const f4 &v) {
  return I == 0 ? v.x : I == 1 ? v.y : I == 2 ? v.z : v.w;
}

template <int I, int TM, int TN>
__device__ __forceinline__ void mfma_step(v16f (&acc)[TM][TN], const f4 (&fa)[TM], const f4 (&fb)[TN]) {
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b)
      acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp<I>(fa[a]), comp<I>(fb[b]), acc[a][b], 0, 0, 0);
}

template <int TM, int TN>
__device__ __forceinline__ void mfma_group(v16f (&acc)[TM][TN], const f4 (&fa)[TM], const f4 (&fb)[TN]) {
  mfma_step<0>(acc, fa, fb);
  mfma_step<1>(acc, fa, fb);
  mfma_step<2>(acc, fa, fb);
  mfma_step<3>(acc, fa, fb);
}

// Loader for whole K steps: no bounds tests.  Rows (and columns) that fall outside the matrix are
// clamped to the last valid one -- they only feed accumulators that the epilogue never stores --
// so every tile, edge tiles included, streams its operands with straight-line loads.  An f4 that
// lies wholly inside its row is fetched with one 16-byte load whatever its alignment (global
// loads only need dword alignment, so leading dimensions like k*k*d = 363 cost nothing extra);
// `vec` = 0 forces four dword loads.  The last f4 of a row-contiguous operand whose row count is
// not a multiple of 4 is assembled from clamped dword loads.
// COLS (row-contiguous operands of the batched kernels only): the columns are numbered across images (ImageCols);
// an f4 that runs over the end of an image continues `skip` floats further on from element `jmp` onward.
template <class T, bool KC, int ROWS, bool COLS = false>
struct FastLoader {
  using L = OperandLayout<T, KC, ROWS>;
  static constexpr int NV = L::NV;
  const float *p[NV];
  int lim[NV];  // row-contiguous scalar mode: element j of the f4 sits at offset min(j, lim)
  int jmp[COLS ? NV : 1];  // COLS: first element of the f4 that lies in the next image (4: none)
  size_t skip;             // COLS: floats between the end of one image's row and the start of the next image's
  size_t step;  // floats per K step
  bool last_active;  // whether this lane owns the (possibly partial) last slot
  __device__ __forceinline__ void init(const float *g, int ld, int row0, int k0, int rows_total, int tid,
                                       const ImageCols *ic = nullptr) {
    last_active = L::active(NV - 1, tid);
    skip = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      // lanes without the last slot point it at their first f4: valid memory, never loaded
      const int f = L::active(i, tid) ? tid + i * T::THREADS : tid;
      if (KC) {
        const int row = min(row0 + f / (T::BK / 4), rows_total - 1), kq = f % (T::BK / 4);
        p[i] = g + (size_t)row * ld + k0 + kq * 4;
        lim[i] = 3;
      } else {
        const int kk = f / (ROWS / 4), rq = f % (ROWS / 4);
        // an f4 starting past the end moves back to the last one that fits
        int start = row0 + rq * 4;
        lim[i] = min(3, rows_total - 1 - start);
        if (lim[i] < 0) {
          start = max(rows_total - 4, 0);
          lim[i] = min(3, rows_total - 1 - start);
        }
        if (COLS && ic && ic->plane) {
          const uint32_t img = fdiv((uint32_t)start, ic->div), px = (uint32_t)start - img * ic->plane;
          p[i] = g + (size_t)(k0 + kk) * ld + (size_t)img * ic->stride + px;
          jmp[i] = (int)min(4u, ic->plane - px);
          skip = ic->stride - ic->plane;
        } else {
          p[i] = g + (size_t)(k0 + kk) * ld + start;
          if (COLS) jmp[i] = 4;
        }
      }
    }
    step = KC ? (size_t)T::BK : (size_t)T::BK * ld;
  }
  __device__ __forceinline__ void load(f4 *__restrict__ r, int vec) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i == NV - 1 && !last_active) continue;
      if (vec && (KC || (lim[i] == 3 && (!COLS || jmp[i] >= 4)))) {
        r[i] = *reinterpret_cast<const f4u *>(p[i]);
      } else if (KC) {
        r[i] = f4{p[i][0], p[i][1], p[i][2], p[i][3]};
      } else if (COLS) {
        const int l = lim[i], j0 = jmp[i];
        const int e1 = min(1, l), e2 = min(2, l), e3 = min(3, l);
        // (an image holds at least one pixel: with planes below four floats an f4 can span three images, which
        // the host excludes)
        r[i] = f4{p[i][0], p[i][e1 + (e1 >= j0 ? skip : 0)], p[i][e2 + (e2 >= j0 ? skip : 0)],
                  p[i][e3 + (e3 >= j0 ? skip : 0)]};
      } else {
        const int l = lim[i];
        r[i] = f4{p[i][0], p[i][min(1, l)], p[i][min(2, l)], p[i][min(3, l)]};
      }
      p[i] += step;
    }
  }
};

// Main K loop of one macro tile.  Whole K steps go through FastLoader; only a partial last step
// (K not a multiple of 16) uses the guarded, zero-filling loader.
//
// Software pipeline (BK = 16 = two k-groups of 8, two LDS stages, ONE barrier per K step):
//   step t, first half : MFMAs of k-group 0 of stage t (fragments fetched during step t-1);
//                        meanwhile the global data of tile t+1 (requested during step t-1) is
//                        written to stage t+1 and the loads of tile t+2 are issued
//   barrier            : stage t+1 is complete, nobody reads stage t any more
//   step t, second half: fragments of k-group 0 of stage t+1 are requested, MFMAs of k-group 1
//                        of stage t run, then the fragments of k-group 1 of stage t+1 are requested
// so LDS and HBM latencies are covered by 32 MFMAs (2048 matrix-pipe cycles) each.
template <class T, bool A_KC, bool B_KC, bool COLS = false>
__device__ __forceinline__ void gemm_mainloop(const GemmArgs &g, const float *__restrict__ Ap,
                                              const float *__restrict__ Bp, float *smem, v16f (&acc)[T::TM][T::TN], int m0,
                                              int n0, int kbeg, int kend, int nk, int tid, int lane, int wm0,
                                              int wn0, const ImageCols *ic = nullptr) {
  using LA = OperandLayout<T, A_KC, T::BM>;
  using LB = OperandLayout<T, B_KC, T::BN>;
  constexpr int STAGE = LA::SIZE + LB::SIZE;  // stage s: A at smem + s*STAGE, B right after it
  static_assert(T::BK == 16, "the pipeline below is written for two k-groups per K step");
  f4 ra[LA::NV], rb[LB::NV];
  FastLoader<T, A_KC, T::BM> la;
  FastLoader<T, B_KC, T::BN, COLS && !B_KC> lb;
  la.init(Ap, g.lda, m0, kbeg, g.M, tid);
  lb.init(Bp, g.ldb, n0, kbeg, g.N, tid, COLS ? ic : nullptr);
  const int nk_full = (kend - kbeg) / T::BK;
// global -> registers for K step t
#define CCT_FETCH(t)                                                                         \
  do {                                                                                       \
    if ((t) >= nk_full) {                                                                    \
      const int k0_ = kbeg + (t) * T::BK;                                                    \
      load_tile<T, A_KC, T::BM>(ra, Ap, g.lda, m0, k0_, g.M, kend, 0, tid);                  \
      load_tile<T, B_KC, T::BN>(rb, Bp, g.ldb, n0, k0_, g.N, kend, 0, tid, COLS ? ic : nullptr); \
    } else {                                                                                 \
      la.load(ra, g.a_vec);                                                                  \
      lb.load(rb, g.b_vec);                                                                  \
    }                                                                                        \
  } while (0)
// registers -> LDS stage
#define CCT_STASH(stage)                                                                     \
  do {                                                                                       \
    store_tile<T, A_KC, T::BM>(smem + (stage) * STAGE, ra, tid);                             \
    store_tile<T, B_KC, T::BN>(smem + (stage) * STAGE + LA::SIZE, rb, tid);                  \
  } while (0)
// LDS stage, k-group -> MFMA fragments
#define CCT_FRAGS(stage, kg, fa, fb)                                                         \
  do {                                                                                       \
    load_frags<T, A_KC, T::BM, T::TM>(fa, smem + (stage) * STAGE, wm0, kg, lane);            \
    load_frags<T, B_KC, T::BN, T::TN>(fb, smem + (stage) * STAGE + LA::SIZE, wn0, kg, lane); \
  } while (0)

  f4 fa0[T::TM], fb0[T::TN], fa1[T::TM], fb1[T::TN];
  if (nk <= 0) return;
  CCT_FETCH(0);
  CCT_STASH(0);
  if (nk > 1) CCT_FETCH(1);
  __syncthreads();
  CCT_FRAGS(0, 0, fa0, fb0);
  CCT_FRAGS(0, 1, fa1, fb1);
  for (int t = 0; t < nk; ++t) {
    const int cur = t & 1;
    const bool more = (t + 1 < nk);
    __builtin_amdgcn_sched_barrier(0);
    mfma_group<T::TM, T::TN>(acc, fa0, fb0);
    if (more) {
      CCT_STASH(cur ^ 1);
      if (t + 2 < nk) CCT_FETCH(t + 2);
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    if (more) CCT_FRAGS(cur ^ 1, 0, fa0, fb0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_group<T::TM, T::TN>(acc, fa1, fb1);
    if (more) CCT_FRAGS(cur ^ 1, 1, fa1, fb1);
  }
#undef CCT_FETCH
#undef CCT_STASH
#undef CCT_FRAGS
}

// ---- operand tiles straight from global memory into LDS ------------------------------------------
// Staging a tile through registers (global load, wait, ds_write) costs the wavefronts instruction
// slots that the matrix pipe does not hide: with the MFMAs taken out, fetching and stashing alone
// took 0.40 ms of the 1.98 ms forward GEMM of the AlexNet conv2 shape.  Here the tiles are moved by
// 16-byte buffer loads that write LDS directly (one instruction moves 64 consecutive 16-byte
// vectors of a stage; each lane supplies the global address of its vector).  LDS rows carry no
// padding -- the transfer cannot insert any -- so a K-contiguous operand stores vector kq of row
// `row` in slot kq ^ ((row >> 1) & 3) of its 4-slot row: eight consecutive rows of one fragment
// read then cover all 32 banks.  Preconditions (checked on the host, else the register path runs):
// operand bases 16-byte aligned, leading dimensions multiples of 4, a row-contiguous operand's row
// count a multiple of 4, K a multiple of 16, operands below 2 GiB (32-bit buffer offsets).
template <class T, bool KC, int ROWS>
struct DmaLayout {
  static constexpr int SIZE = ROWS * T::BK;       // floats per stage
  static constexpr int TOTAL = ROWS * T::BK / 4;  // 16-byte vectors per stage
  static constexpr int NWAVES = T::THREADS / 64;
  static constexpr int NV = (TOTAL / 64 + NWAVES - 1) / NWAVES;  // transfers per wavefront per stage
  // byte offset of the vector that lane `lane` of wavefront `wave` moves in transfer i, for K step 0
  static __device__ __forceinline__ uint32_t source(int i, int wave, int lane, int row0, int rows_total, int ld) {
    const int f = (i * NWAVES + wave) * 64 + lane;
    if (KC) {
      const int row = f >> 2, slot = f & 3, kq = slot ^ ((row >> 1) & 3);
      return (uint32_t)(min(row0 + row, rows_total - 1) * (size_t)ld + kq * 4) * 4u;
    }
    const int kk = f / (ROWS / 4), rq = f - kk * (ROWS / 4);
    return (uint32_t)((size_t)kk * ld + min(row0 + rq * 4, rows_total - 4)) * 4u;
  }
  // the same for a row-contiguous operand whose columns are numbered across images (the plane a multiple of 4
  // floats: a vector never runs over the end of an image)
  static __device__ __forceinline__ uint32_t source_cols(int i, int wave, int lane, int row0, int rows_total, int ld,
                                                         const ImageCols &ic) {
    const int f = (i * NWAVES + wave) * 64 + lane;
    const int kk = f / (ROWS / 4), rq = f - kk * (ROWS / 4);
    return (uint32_t)((size_t)kk * ld + ic.offset((uint32_t)min(row0 + rq * 4, rows_total - 4))) * 4u;
  }
};

template <class T, bool KC, int ROWS, int NT>
struct DmaFrags {
  // per-lane LDS offsets (floats) of the fragments of k-group 0 and 1 for the tile at wave row `wrow0`
  int base[2];
  __device__ __forceinline__ void init(int wrow0, int lane) {
    const int r = lane & 31, h = lane >> 5;
    if (KC) {
      const int sw = (r >> 1) & 3;
      base[0] = (wrow0 + r) * T::BK + ((h ^ sw) << 2);
      base[1] = (wrow0 + r) * T::BK + (((2 + h) ^ sw) << 2);
    } else {
      base[0] = (h * 4) * ROWS + wrow0 + r;
      base[1] = (8 + h * 4) * ROWS + wrow0 + r;
    }
  }
  template <int KG>
  __device__ __forceinline__ void load(f4 (&f)[NT], const float *__restrict__ lds) const {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (KC) {
        f[t] = *reinterpret_cast<const f4 *>(lds + base[KG] + t * 32 * T::BK);
      } else {
        const float *p = lds + base[KG] + t * 32;
        f[t].x = p[0];
        f[t].y = p[ROWS];
        f[t].z = p[2 * ROWS];
        f[t].w = p[3 * ROWS];
      }
    }
  }
};

// Main K loop with direct transfers (K a multiple of BK = 16, two k-groups per step, two LDS
// buffers, one barrier per step in the MIDDLE of the step):
//   step t, first half : MFMAs of k-group 0 of stage t (both k-groups' fragments were read from LDS
//                        during step t-1)
//   wait + barrier     : stage t+1 (requested a whole step ago) has landed, and every wavefront's
//                        reads of stage t have completed, so its buffer is free
//   step t, second half: the transfers of stage t+2 are requested into that buffer, the fragments
//                        of k-group 0 of stage t+1 are requested, MFMAs of k-group 1 of stage t run,
//                        the fragments of k-group 1 of stage t+1 are requested
template <class T, bool A_KC, bool B_KC, bool COLS = false>
__device__ __forceinline__ void gemm_mainloop_dma(const GemmArgs &g, const float *Ap, const float *Bp, float *smem,
                                                  v16f (&acc)[T::TM][T::TN], int m0,
                                                  int n0, int kbeg, int nk, int lane, int wave, int wm0,
                                                  int wn0, const ImageCols *ic = nullptr) {
  using DA = DmaLayout<T, A_KC, T::BM>;
  using DB = DmaLayout<T, B_KC, T::BN>;
  constexpr int STAGE = DA::SIZE + DB::SIZE;
  constexpr int NW = T::THREADS / 64;
  static_assert(T::BK == 16, "two k-groups per K step");
  if (nk <= 0) return;
  uint32_t aoff[DA::NV], boff[DB::NV];
#pragma unroll
  for (int i = 0; i < DA::NV; ++i) aoff[i] = DA::source(i, wave, lane, m0, g.M, g.lda);
#pragma unroll
  for (int i = 0; i < DB::NV; ++i)
    boff[i] = (COLS && !B_KC && ic && ic->plane) ? DB::source_cols(i, wave, lane, n0, g.N, g.ldb, *ic)
                                                 : DB::source(i, wave, lane, n0, g.N, g.ldb);
  const rsrc_t a_rsrc = make_rsrc(Ap), b_rsrc = make_rsrc(Bp);
  const uint32_t a_step = A_KC ? (uint32_t)T::BK * 4u : (uint32_t)T::BK * (uint32_t)g.lda * 4u;
  const uint32_t b_step = B_KC ? (uint32_t)T::BK * 4u : (uint32_t)T::BK * (uint32_t)g.ldb * 4u;
  const uint32_t a_k0 = A_KC ? (uint32_t)kbeg * 4u : (uint32_t)kbeg * (uint32_t)g.lda * 4u;
  const uint32_t b_k0 = B_KC ? (uint32_t)kbeg * 4u : (uint32_t)kbeg * (uint32_t)g.ldb * 4u;
// transfers of K step t -> LDS buffer buf
#define CCT_DMA_ISSUE(t, buf)                                                                      \
  do {                                                                                             \
    float *sa_ = smem + (buf) * STAGE, *sb_ = sa_ + DA::SIZE;                                      \
    const uint32_t ga_ = a_k0 + (uint32_t)(t) * a_step, gb_ = b_k0 + (uint32_t)(t) * b_step;       \
    _Pragma("unroll") for (int i = 0; i < DA::NV; ++i) {                                           \
      if ((i * NW + wave) * 64 < DA::TOTAL) lds_dma16(a_rsrc, aoff[i], ga_, sa_ + (i * NW + wave) * 256); \
    }                                                                                              \
    _Pragma("unroll") for (int i = 0; i < DB::NV; ++i) {                                           \
      if ((i * NW + wave) * 64 < DB::TOTAL) lds_dma16(b_rsrc, boff[i], gb_, sb_ + (i * NW + wave) * 256); \
    }                                                                                              \
  } while (0)
  DmaFrags<T, A_KC, T::BM, T::TM> qa;
  DmaFrags<T, B_KC, T::BN, T::TN> qb;
  qa.init(wm0, lane);
  qb.init(wn0, lane);

  f4 fa0[T::TM], fb0[T::TN], fa1[T::TM], fb1[T::TN];
  CCT_DMA_ISSUE(0, 0);
  if (nk > 1) CCT_DMA_ISSUE(1, 1);
  lds_dma_wait();
  __syncthreads();
  qa.template load<0>(fa0, smem);
  qb.template load<0>(fb0, smem + DA::SIZE);
  qa.template load<1>(fa1, smem);
  qb.template load<1>(fb1, smem + DA::SIZE);
  for (int t = 0; t < nk; ++t) {
    const int cur = t & 1;
    const bool more = (t + 1 < nk);
    __builtin_amdgcn_sched_barrier(0);
    mfma_group<T::TM, T::TN>(acc, fa0, fb0);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): stage t+1 landed; lgkmcnt(0): this wave's reads of stage t are done
    __syncthreads();
    if (t + 2 < nk) CCT_DMA_ISSUE(t + 2, cur);
    const float *nxt = smem + (cur ^ 1) * STAGE;
    if (more) {
      qa.template load<0>(fa0, nxt);
      qb.template load<0>(fb0, nxt + DA::SIZE);
    }
    __builtin_amdgcn_sched_barrier(0);
    mfma_group<T::TM, T::TN>(acc, fa1, fb1);
    if (more) {
      qa.template load<1>(fa1, nxt);
      qb.template load<1>(fb1, nxt + DA::SIZE);
    }
  }
#undef CCT_DMA_ISSUE
}

// Epilogue of a tile whose columns lie wholly inside C and that reads nothing back: per lane one
// row pointer advancing by a row stride and TN fixed column offsets.  ROWGUARD = false: the rows
// lie inside C too, no bounds tests at all; true: rows past M are skipped (M not a multiple of the
// tile height, e.g. 96 output maps).  row0/col0 are the lane's first row and column.
template <class T, int MODE, bool ROWGUARD>
__device__ __forceinline__ void fast_epilogue(const GemmArgs &g, float *Cp, const v16f (&acc)[T::TM][T::TN], int row0,
                                              int col0, uint32_t kslice) {
  if (MODE == EPI_CONV_FORWARD) {
    size_t coff[T::TN];
#pragma unroll
    for (int b = 0; b < T::TN; ++b) {
      const uint32_t col = col0 + b * 32;
      const uint32_t img = fdiv(col, g.div_fmap);
      coff[b] = (size_t)img * g.M * g.fmap + (col - img * g.fmap);
    }
#pragma unroll
    for (int a = 0; a < T::TM; ++a)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = row0 + a * 32 + 8 * j + i;
          if (ROWGUARD && row >= g.M) continue;
          float *c = Cp + (size_t)row * g.fmap;
          const float add = g.bias ? g.bias[row] : 0.0f;
#pragma unroll
          for (int b = 0; b < T::TN; ++b) {
            const float y = acc[a][b][4 * j + i] + add;
            c[coff[b]] = (g.relu && !(y > 0.0f)) ? 0.0f : y;
          }
        }
  } else {
    const size_t rstride = (MODE == EPI_SPLITK_PARTIAL) ? (size_t)g.N : (size_t)g.ldc;
    float *crow = ((MODE == EPI_SPLITK_PARTIAL) ? g.ws + (size_t)kslice * g.M * g.N : Cp) +
                  (size_t)row0 * rstride + col0;
    const float alpha = g.alpha;
    // column bias and clamp of the plain epilogue (a fully connected layer's forward pass); uniform
    const bool post = MODE == EPI_ALPHA_BETA && (g.col_bias || g.relu);
    float cb[T::TN];
#pragma unroll
    for (int b = 0; b < T::TN; ++b) cb[b] = (post && g.col_bias) ? g.col_bias[col0 + b * 32] : 0.0f;
#pragma unroll
    for (int a = 0; a < T::TM; ++a)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (ROWGUARD && row0 + a * 32 + 8 * j + i >= g.M) continue;
          float *c = crow + (size_t)(a * 32 + 8 * j + i) * rstride;
#pragma unroll
          for (int b = 0; b < T::TN; ++b) {
            float y = (MODE == EPI_SPLITK_PARTIAL) ? acc[a][b][4 * j + i] : alpha * acc[a][b][4 * j + i];
            if (post) {
              if (g.col_bias) y += cb[b];
              if (g.relu && !(y > 0.0f)) y = 0.0f;
            }
            c[b * 32] = y;
          }
        }
  }
}

// One workgroup's tile.  BATCHED: a batch of products in one launch (GemmArgs::bmode) -- the matrix pointers move
// with the slice and the main loop sits in a loop over images.  That costs the 128 x 128 instances 30 registers
// (and cost the inner-product GEMMs of CaffeNet 13 % while the plain kernel carried it), so the batched form is a
// template parameter and has kernels of its own.
template <class T, bool A_KC, bool B_KC, bool DMA, bool BATCHED>
__device__ __forceinline__ void gemm_workgroup(const GemmArgs &g, float *smem) {
  const float *Ap = g.A, *Bp = g.B;
  float *Cp = g.C;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / T::WGN) * T::WM, wn0 = (wave % T::WGN) * T::WN;

  // One flat grid over (K slice, tile) with the tile index fastest: the workgroups that share an
  // operand panel (same K slice, neighbouring tiles) get consecutive ids on one XCD and run
  // together.  Within a K slice the dimension with fewer tiles runs fastest.
  const uint32_t flat = xcd_remap(blockIdx.x, g.nblocks);
  const uint32_t kslice = flat / g.ntiles;
  const uint32_t id = flat - kslice * g.ntiles;
  int tm, tn;
  if (g.tiles_m <= g.tiles_n) {
    tm = id % g.tiles_m; tn = id / g.tiles_m;
  } else {
    tn = id % g.tiles_n; tm = id / g.tiles_n;
  }
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  int kbeg = kslice * g.kchunk;
  int more_images = 0;  // bmode 2: images of this slice after the first
  ImageCols ic{0u, g.div_bplane, 0};
  if constexpr (BATCHED) {
    if (g.bmode == 3) {
      ic.plane = g.bplane;
      ic.stride = g.b_bstride;
    } else {
      const uint32_t igroup = g.bmode == 1 ? kslice : kslice / (uint32_t)g.bksplit;
      kbeg = g.bmode == 1 ? 0 : (int)(kslice - igroup * g.bksplit) * g.kchunk;
      const uint32_t img = g.bmode == 1 ? igroup : igroup * (uint32_t)g.bgroup;
      Ap += (size_t)img * g.a_bstride;
      Bp += (size_t)img * g.b_bstride;
      if (g.bmode == 1) Cp += (size_t)img * g.c_bstride;
      else more_images = min(g.bgroup, g.nbatch - (int)img) - 1;
    }
  }
  const int kend = min(g.K, kbeg + g.kchunk);
  const int nk = (kend - kbeg + T::BK - 1) / T::BK;

  v16f acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  if constexpr (BATCHED) {
    for (;;) {
      if (DMA) gemm_mainloop_dma<T, A_KC, B_KC, true>(g, Ap, Bp, smem, acc, m0, n0, kbeg, nk, lane, __builtin_amdgcn_readfirstlane(wave), wm0, wn0, &ic);
      else gemm_mainloop<T, A_KC, B_KC, true>(g, Ap, Bp, smem, acc, m0, n0, kbeg, kend, nk, tid, lane, wm0, wn0, &ic);
      if (--more_images < 0) break;
      // the next image of the sum: same tile, same accumulators; the LDS stages are refilled from scratch
      Ap += g.a_bstride;
      Bp += g.b_bstride;
      __syncthreads();
    }
  } else {
    if (DMA) gemm_mainloop_dma<T, A_KC, B_KC>(g, Ap, Bp, smem, acc, m0, n0, kbeg, nk, lane, __builtin_amdgcn_readfirstlane(wave), wm0, wn0);
    else gemm_mainloop<T, A_KC, B_KC>(g, Ap, Bp, smem, acc, m0, n0, kbeg, kend, nk, tid, lane, wm0, wn0);
  }
  const bool rows_inside = m0 + T::BM <= g.M, cols_inside = n0 + T::BN <= g.N;

  // epilogue: accumulator register v of lane (r,h) is C[8*(v/4) + 4*h + v%4][r] of its 32x32 tile
  const int r = lane & 31, h = lane >> 5;
  if (cols_inside && !(g.epi == EPI_ALPHA_BETA && g.beta != 0.0f)) {
    const int er = m0 + wm0 + 4 * h, ec = n0 + wn0 + r;
    if (rows_inside) {
      if (g.epi == EPI_ALPHA_BETA) fast_epilogue<T, EPI_ALPHA_BETA, false>(g, Cp, acc, er, ec, kslice);
      else if (g.epi == EPI_SPLITK_PARTIAL) fast_epilogue<T, EPI_SPLITK_PARTIAL, false>(g, Cp, acc, er, ec, kslice);
      else fast_epilogue<T, EPI_CONV_FORWARD, false>(g, Cp, acc, er, ec, kslice);
    } else {
      if (g.epi == EPI_ALPHA_BETA) fast_epilogue<T, EPI_ALPHA_BETA, true>(g, Cp, acc, er, ec, kslice);
      else if (g.epi == EPI_SPLITK_PARTIAL) fast_epilogue<T, EPI_SPLITK_PARTIAL, true>(g, Cp, acc, er, ec, kslice);
      else fast_epilogue<T, EPI_CONV_FORWARD, true>(g, Cp, acc, er, ec, kslice);
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < T::TN; ++b) {
    const int col = n0 + wn0 + b * 32 + r;
    if (col >= g.N) continue;
    size_t col_off;
    if (g.epi == EPI_CONV_FORWARD) {
      const uint32_t img = fdiv((uint32_t)col, g.div_fmap);
      col_off = (size_t)img * g.M * g.fmap + (col - img * g.fmap);
    } else {
      col_off = col;
    }
#pragma unroll
    for (int a = 0; a < T::TM; ++a) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm0 + a * 32 + 8 * (v / 4) + 4 * h + (v % 4);
        if (row >= g.M) continue;
        const float x = acc[a][b][v];
        if (g.epi == EPI_ALPHA_BETA) {
          float *c = Cp + (size_t)row * g.ldc + col_off;
          float y = (g.beta == 0.0f) ? g.alpha * x : g.alpha * x + g.beta * (*c);
          if (g.col_bias) y += g.col_bias[col];
          if (g.relu && !(y > 0.0f)) y = 0.0f;
          if (g.nt_store) __builtin_nontemporal_store(y, c);
          else *c = y;
        } else if (g.epi == EPI_SPLITK_PARTIAL) {
          g.ws[((size_t)kslice * g.M + row) * g.N + col_off] = x;
        } else {
          float y = g.bias ? x + g.bias[row] : x;
          if (g.relu && !(y > 0.0f)) y = 0.0f;
          if (g.nt_store) __builtin_nontemporal_store(y, Cp + (size_t)row * g.fmap + col_off);
          else Cp[(size_t)row * g.fmap + col_off] = y;
        }
      }
    }
  }
}

template <class T, bool A_KC, bool B_KC, bool DMA = false>
__global__ __launch_bounds__(T::THREADS, 2) void gemm_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float smem[2 * (OperandLayout<T, A_KC, T::BM>::SIZE + OperandLayout<T, B_KC, T::BN>::SIZE)];
  gemm_workgroup<T, A_KC, B_KC, DMA, false>(g, smem);
}

// The same tile code for a batch of products in one launch (GemmArgs::bmode: 1 x 1 convolutions).
template <class T, bool A_KC, bool B_KC, bool DMA = false>
__global__ __launch_bounds__(T::THREADS, 2) void gemm_batched_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float smem[2 * (OperandLayout<T, A_KC, T::BM>::SIZE + OperandLayout<T, B_KC, T::BN>::SIZE)];
  gemm_workgroup<T, A_KC, B_KC, DMA, true>(g, smem);
}

// C = alpha * sum_z ws[z] + beta * C, z ascending (fixed order); then the optional column bias and clamp.
// fmap > 0: the epilogue of the forward convolution instead (output permutation, bias per row, clamp).
// Workgroups from `cs_first` on do an unrelated small job that rides along in this launch: the column sums of
// cs.src (colsum.h).
struct ColSumJob {
  float *dst;
  const float *src;
  int rows, cols;
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(float *__restrict__ C,
                                                            const float *__restrict__ ws, int M, int N,
                                                            int ldc, int splits, float alpha, float beta,
                                                            FastDiv div_n, const float *__restrict__ col_bias,
                                                            int relu, const float *__restrict__ row_bias, int fmap,
                                                            FastDiv div_fmap, uint32_t cs_first, ColSumJob cs) {
  __shared__ float cs_part[4][64];
  if (blockIdx.x >= cs_first) {  // workgroup-uniform
    colsum_block(cs.dst, cs.src, cs.cols, cs.rows, blockIdx.x - cs_first, cs_part);
    return;
  }
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= (uint32_t)M * N) return;
  const uint32_t row = fdiv(e, div_n);
  const uint32_t col = e - row * N;
  float s = 0.0f;
  const size_t mn = (size_t)M * N;
  const float *p = ws + e;
  int z = 0;
  // eight partial sums in flight per lane; added in slice order
  for (; z + 8 <= splits; z += 8, p += 8 * mn) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[(size_t)j * mn];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
  for (; z < splits; ++z, p += mn) s += *p;
  if (fmap > 0) {
    // forward convolution: C is [image][row][fmap], column = image * fmap + position; bias per row
    const uint32_t img = fdiv(col, div_fmap);
    float y = row_bias ? s + row_bias[row] : s;
    if (relu && !(y > 0.0f)) y = 0.0f;
    C[((size_t)img * M + row) * fmap + (col - img * fmap)] = y;
    return;
  }
  float *c = C + (size_t)row * ldc + col;
  float y = (beta == 0.0f) ? alpha * s : alpha * s + beta * (*c);
  if (col_bias) y += col_bias[col];
  if (relu && !(y > 0.0f)) y = 0.0f;
  *c = y;
}

typedef Tile<256, 128, 16, 2, 2> TileL;
typedef Tile<128, 256, 16, 2, 2> TileLT;  // same wave work as TileL with the long side along N
typedef Tile<128, 128, 16, 2, 2> TileM;
typedef Tile<64, 64, 16, 2, 2> TileS;
// 96 rows (AlexNet conv1's 96 output maps would waste a quarter of a 128-row tile): the four
// wavefronts sit side by side, each owning 96 x 32
typedef Tile<96, 128, 16, 1, 4> TileR;

template <class T>
static int launch_cfg(GemmArgs &g, bool a_kc, bool b_kc, int splits, hipStream_t st) {
  g.tiles_m = (g.M + T::BM - 1) / T::BM;
  g.tiles_n = (g.N + T::BN - 1) / T::BN;
  g.ntiles = (uint32_t)g.tiles_m * g.tiles_n;
  g.splits = splits;
  const size_t nblocks = (size_t)g.ntiles * splits;
  if (nblocks >= (1ull << 31)) return set_error(CCT_HIP_EINVAL, "sgemm: too many workgroups");
  g.nblocks = (uint32_t)nblocks;
  dim3 grid(g.nblocks), block(T::THREADS);
  if (g.bmode) {
    // the batched products of the 1 x 1 layers: forward (A K-contiguous, B row-contiguous), data gradient (both
    // row-contiguous), weight gradient (both K-contiguous)
    if (a_kc && !b_kc) {
      if (g.dma) hipLaunchKernelGGL((gemm_batched_kernel<T, true, false, true>), grid, block, 0, st, g);
      else hipLaunchKernelGGL((gemm_batched_kernel<T, true, false>), grid, block, 0, st, g);
    } else if (!a_kc && !b_kc) {
      if (g.dma) hipLaunchKernelGGL((gemm_batched_kernel<T, false, false, true>), grid, block, 0, st, g);
      else hipLaunchKernelGGL((gemm_batched_kernel<T, false, false>), grid, block, 0, st, g);
    } else if (a_kc && b_kc) {
      if (g.dma) hipLaunchKernelGGL((gemm_batched_kernel<T, true, true, true>), grid, block, 0, st, g);
      else hipLaunchKernelGGL((gemm_batched_kernel<T, true, true>), grid, block, 0, st, g);
    } else {
      return set_error(CCT_HIP_EINVAL, "sgemm: no batched instance for these operand layouts");
    }
  } else if (g.dma) {
    if (a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, true, true>), grid, block, 0, st, g);
    else if (a_kc && !b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, false, true>), grid, block, 0, st, g);
    else if (!a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, false, true, true>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_kernel<T, false, false, true>), grid, block, 0, st, g);
  } else {
    if (a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, true>), grid, block, 0, st, g);
    else if (a_kc && !b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, false>), grid, block, 0, st, g);
    else if (!a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, false, true>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_kernel<T, false, false>), grid, block, 0, st, g);
  }
  CCT_LAUNCH_CHECK();
  note_kernel("%s<Tile<%d,%d,%d,%d,%d>,%s,%s%s> splits=%d", g.bmode ? "gemm_batched_kernel" : "gemm_kernel", T::BM,
              T::BN, T::BK, T::WGM, T::WGN, a_kc ? "true" : "false", b_kc ? "true" : "false", g.dma ? ",true" : "",
              splits);
  return 0;
}

// Row-major GEMM driver.  a_kc: A(m,k) = A[m*lda + k] (cblas NoTrans); b_kc: B(k,n) = B[n*ldb + k]
// (cblas Trans).
__global__ __launch_bounds__(256) void colsum_kernel(ColSumJob cs) {
  __shared__ float part[4][64];
  colsum_block(cs.dst, cs.src, cs.cols, cs.rows, blockIdx.x, part);
}

// A batch of products in one launch (GemmArgs::bmode): `count` images, strides in floats between them.
struct GemmBatch {
  int mode, count;
  size_t a_stride, b_stride, c_stride;
};

// `colsum`: column sums to compute beside the product, in the spare workgroups of the split-K reduction when
// there is one, else in a launch of their own.  `batch`: M, N, K and the matrices describe one image.
static int gemm_rowmajor(bool a_kc, bool b_kc, int M, int N, int K, float alpha, const float *A, int lda,
                         const float *B, int ldb, float beta, float *C, int ldc, int epi, int fmap,
                         const float *bias, int relu = 0, const float *col_bias = nullptr,
                         const ColSumJob *colsum = nullptr, const GemmBatch *batch = nullptr) {
  if (M <= 0 || N <= 0) {
    if (colsum && colsum->cols > 0) {
      hipLaunchKernelGGL(colsum_kernel, dim3((uint32_t)((colsum->cols + 63) / 64)), dim3(256), 0, ctx().stream, *colsum);
      CCT_LAUNCH_CHECK();
    }
    return 0;
  }
  hipStream_t st = ctx().stream;
  GemmArgs g;
  g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.alpha = alpha; g.beta = beta; g.epi = epi; g.fmap = fmap > 0 ? fmap : 1;
  g.div_fmap = make_fastdiv((uint32_t)g.fmap); g.bias = bias; g.relu = relu; g.col_bias = col_bias; g.ws = nullptr;
  // 16-byte global loads need dword alignment only
  g.a_vec = ((uintptr_t)A % 4 == 0);
  g.b_vec = ((uintptr_t)B % 4 == 0);
  g.nt_store = tuning().gemm_nt;
  if (K <= 0) g.K = 0;  // degenerate: C = beta*C through the normal epilogue with zero accumulators
  const int bmode = batch ? batch->mode : 0, nbatch = batch ? batch->count : 1;
  g.bmode = bmode; g.nbatch = nbatch; g.bgroup = 1; g.bksplit = 1;
  g.a_bstride = batch ? batch->a_stride : 0; g.b_bstride = batch ? batch->b_stride : 0;
  g.c_bstride = batch ? batch->c_stride : 0;
  g.bplane = bmode == 3 ? (uint32_t)g.fmap : 1u;
  g.div_bplane = make_fastdiv(g.bplane);

  // Tile shape and split-K factor come from a small occupancy model.  A compute unit holds `occ`
  // workgroups of a shape; the busiest unit gets n = ceil(blocks / units) of them and works them off
  // in groups of occ.  A group of j co-resident workgroups runs at min(j * 0.55, 1) of the unit's
  // MFMA rate (one workgroup alone cannot hide its own barriers), every workgroup pays a fixed
  // prologue/epilogue worth `k0` K-steps, and the smaller shapes lose a little to their lower
  // flop-per-LDS-byte ratio (`eff`).  The constants are fitted to measured times of the
  // AlexNet/CaffeNet convolution and inner-product shapes.
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  const int bk = 16;
  struct Shape { int bm, bn, occ, k0; double eff; };
  static const Shape shapes_plain[5] = {{256, 128, 2, 32, 1.0}, {128, 128, 3, 8, 0.96}, {64, 64, 6, 8, 0.80},
                                        {128, 256, 2, 32, 1.0}, {96, 128, 3, 8, 0.90}};  // L, M, S, LT, R
  // Products per image (1 x 1 layers) have short contractions -- the channel count, or one image's pixels -- and
  // every image is a pipeline of its own to fill and drain: fitted to all five shapes timed on 107 layers (7 x 7
  // to 56 x 56 maps, 64 to 1024 channels and maps, batch 32 and 128; forward, data and weight gradient), the
  // fixed cost per workgroup is several times that of the long products above and the small tile loses less.
  // Mean time over the best shape's 1.003 (worst 1.09); the constants above gave 1.028 (worst 1.42).
  static const Shape shapes_batched[5] = {{256, 128, 2, 96, 1.0}, {128, 128, 3, 48, 0.90}, {64, 64, 6, 16, 0.90},
                                          {128, 256, 2, 96, 1.0}, {96, 128, 3, 48, 1.0}};
  const Shape *shapes = bmode ? shapes_batched : shapes_plain;
  const double solo = bmode ? 0.45 : 0.55;  // share of the unit's rate one workgroup reaches alone
  const double cu_rate = 0.8 * 157.3e12 / 256.0, hbm_rate = 4.0e12;
  int cfg = 1, splits = 1, kchunk = g.K > 0 ? g.K : bk;
  double best = 1e30;
  const int forced = tuning().gemm_tile;
  for (int c = 0; c < 5; ++c) {
    if (forced >= 0 && forced <= 4 && c != forced) continue;  // tuning override
    const Shape &sh = shapes[c];
    const long tiles = (long)((M + sh.bm - 1) / sh.bm) * ((N + sh.bn - 1) / sh.bn) * (bmode == 1 ? nbatch : 1);
    const long slots = (long)sh.occ * cus;
    if (bmode == 2) {
      // one product summed over the images: the slices are groups of images or, when there are fewer images than
      // slices wanted, K ranges of single images -- as many as fill the device while a slice keeps some 256 of
      // K; every image refills the pipeline (about four K steps' worth)
      long sp = tiles >= slots ? 1 : slots / tiles;
      const long most = ((long)nbatch * K + 255) / 256;
      if (sp > most) sp = most;
      if (sp < 1) sp = 1;
      int group = 1, ksplit = 1, kc = K > 0 ? K : bk;
      if (sp <= nbatch) {
        group = (int)((nbatch + sp - 1) / sp);
      } else {
        ksplit = (int)(sp / nbatch);
        kc = (((K + ksplit - 1) / ksplit) + bk - 1) / bk * bk;
        ksplit = (K + kc - 1) / kc;
      }
      sp = (long)((nbatch + group - 1) / group) * ksplit;
      const long blocks = tiles * sp, n = (blocks + cus - 1) / cus, rem = n % sh.occ;
      const double w = 2.0 * sh.bm * sh.bn * ((double)group * (kc + 4 * bk) + sh.k0) / (cu_rate * sh.eff);
      double t = (double)(n / sh.occ) * sh.occ * w;
      if (rem) t += rem * w / (rem * solo < 1.0 ? rem * solo : 1.0);
      if (sp > 1) t += 5e-6 + 8.0 * sp * (double)M * N / hbm_rate;
      if (t < best) { best = t; cfg = c; splits = (int)sp; kchunk = kc; g.bgroup = group; g.bksplit = ksplit; }
      continue;
    }
    for (int pass = 0; pass < 2; ++pass) {
      int sp = 1, kc = g.K > 0 ? g.K : bk;
      if (pass == 1) {
        if (bmode) break;
        // split-K, when the tile grid alone cannot fill the device (the reduction then carries the epilogue)
        // (K slices of at least 256, or 128 when the result is small enough for a cheap reduction:
        // those problems are bound by the latency of their few K steps, not by throughput)
        const int min_chunk = (size_t)M * N <= 262144 ? 128 : 256;
        if (tiles >= slots || K < 2 * min_chunk) break;
        sp = (int)(slots / tiles);
        if (sp > K / min_chunk) sp = K / min_chunk;
        if (sp < 2) break;
        kc = (((K + sp - 1) / sp) + bk - 1) / bk * bk;
        sp = (K + kc - 1) / kc;
        if (sp < 2) break;
      }
      const long blocks = tiles * sp;
      const long n = (blocks + cus - 1) / cus;
      const double w = 2.0 * sh.bm * sh.bn * (double)(kc + sh.k0) / (cu_rate * sh.eff);
      const long rem = n % sh.occ;
      double t = (double)(n / sh.occ) * sh.occ * w;
      if (rem) t += rem * w / (rem * solo < 1.0 ? rem * solo : 1.0);
      if (sp > 1) t += 5e-6 + 8.0 * sp * (double)M * N / hbm_rate;  // partial sums out and back in
      if (t < best) { best = t; cfg = c; splits = sp; kchunk = kc; }
    }
  }
  g.kchunk = kchunk;
  {
    // direct global -> LDS transfers need aligned, 4-float-granular operands below 2 GiB and whole K steps
    const size_t a_floats = a_kc ? (size_t)M * lda : (size_t)g.K * lda,
                 b_floats = bmode == 3 ? (size_t)nbatch * g.b_bstride : b_kc ? (size_t)N * ldb : (size_t)g.K * ldb;
    g.dma = g.K > 0 && g.K % bk == 0 && kchunk % bk == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)B % 16 == 0 &&
            lda % 4 == 0 && ldb % 4 == 0 && (a_kc || M % 4 == 0) && (b_kc || N % 4 == 0) &&
            a_floats < (1ull << 29) && b_floats < (1ull << 29) && !tuning().gemm_nodma &&
            g.a_bstride % 4 == 0 && g.b_bstride % 4 == 0;
  }
  const int slices = bmode == 1 ? nbatch : splits;  // what the grid multiplies the tiles by
  if (splits > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)splits * M * N * sizeof(float), &ws);
    if (rc) return rc;
    g.ws = (float *)ws;
    g.epi = EPI_SPLITK_PARTIAL;
  }
  int rc = cfg == 0   ? launch_cfg<TileL>(g, a_kc, b_kc, slices, st)
           : cfg == 1 ? launch_cfg<TileM>(g, a_kc, b_kc, slices, st)
           : cfg == 2 ? launch_cfg<TileS>(g, a_kc, b_kc, slices, st)
           : cfg == 3 ? launch_cfg<TileLT>(g, a_kc, b_kc, slices, st)
                      : launch_cfg<TileR>(g, a_kc, b_kc, slices, st);
  if (rc) return rc;
  if (splits > 1) {
    CCT_REQUIRE((size_t)M * N < (1ull << 31), "sgemm: split-K result too large");
    const uint32_t blocks = (uint32_t)(((size_t)M * N + 255) / 256);
    const uint32_t extra = colsum && colsum->cols > 0 ? (uint32_t)((colsum->cols + 63) / 64) : 0u;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks + extra), dim3(256), 0, st, C, g.ws, M, N, ldc, splits,
                       alpha, beta, make_fastdiv((uint32_t)N), col_bias, relu, bias,
                       epi == EPI_CONV_FORWARD ? g.fmap : 0, g.div_fmap, blocks,
                       colsum ? *colsum : ColSumJob{nullptr, nullptr, 0, 0});
    CCT_LAUNCH_CHECK();
  } else if (colsum && colsum->cols > 0) {
    hipLaunchKernelGGL(colsum_kernel, dim3((uint32_t)((colsum->cols + 63) / 64)), dim3(256), 0, st, *colsum);
    CCT_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_sgemm(int order, int TA, int TB, int M, int N, int K, float alpha, const float *A,
                             int lda, const float *B, int ldb, float beta, float *C, int ldc) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(order == CCT_ROW_MAJOR || order == CCT_COL_MAJOR, "sgemm: bad order %d", order);
  CCT_REQUIRE((TA == CCT_NO_TRANS || TA == CCT_TRANS) && (TB == CCT_NO_TRANS || TB == CCT_TRANS),
              "sgemm: bad transpose flags %d %d", TA, TB);
  CCT_REQUIRE(M >= 0 && N >= 0 && K >= 0, "sgemm: negative dimension");
  if (M == 0 || N == 0) return 0;
  CCT_REQUIRE(A && B && C, "sgemm: null matrix");
  if (order == CCT_COL_MAJOR) {
    // C^T = op(B)^T * op(A)^T : the same memory read as row-major with the operands swapped
    const int rowsA = (TA == CCT_NO_TRANS) ? M : K, rowsB = (TB == CCT_NO_TRANS) ? K : N;
    CCT_REQUIRE(lda >= (rowsA > 1 ? rowsA : 1) && ldb >= (rowsB > 1 ? rowsB : 1) && ldc >= (M > 1 ? M : 1),
                "sgemm: leading dimension too small");
    return gemm_rowmajor(TB == CCT_NO_TRANS, TA == CCT_TRANS, N, M, K, alpha, B, ldb, A, lda, beta, C, ldc,
                         EPI_ALPHA_BETA, 0, nullptr);
  }
  const int colsA = (TA == CCT_NO_TRANS) ? K : M, colsB = (TB == CCT_NO_TRANS) ? N : K;
  CCT_REQUIRE(lda >= (colsA > 1 ? colsA : 1) && ldb >= (colsB > 1 ? colsB : 1) && ldc >= (N > 1 ? N : 1),
              "sgemm: leading dimension too small");
  return gemm_rowmajor(TA == CCT_NO_TRANS, TB == CCT_TRANS, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc,
                       EPI_ALPHA_BETA, 0, nullptr);
}

extern "C" int cct_hip_sgemm_new(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                                 const float *B, float beta, float *C) {
  const int lda = (TA == CCT_NO_TRANS) ? K : M;
  const int ldb = (TB == CCT_NO_TRANS) ? N : K;
  return cct_hip_sgemm(CCT_ROW_MAJOR, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, C, N);
}

extern "C" int cct_hip_sgemm_new_colsum(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                                        const float *B, float beta, float *C, float *colsum, const float *colsum_src,
                                        int rows, int cols) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE((TA == CCT_NO_TRANS || TA == CCT_TRANS) && (TB == CCT_NO_TRANS || TB == CCT_TRANS),
              "sgemm_new_colsum: bad transpose flags %d %d", TA, TB);
  CCT_REQUIRE(M >= 0 && N >= 0 && K >= 0 && rows >= 0 && cols >= 0, "sgemm_new_colsum: negative dimension");
  CCT_REQUIRE((M == 0 || N == 0) || (A && B && C), "sgemm_new_colsum: null matrix");
  CCT_REQUIRE(cols == 0 || (colsum && colsum_src), "sgemm_new_colsum: null column-sum argument");
  const int lda = (TA == CCT_NO_TRANS) ? K : M;
  const int ldb = (TB == CCT_NO_TRANS) ? N : K;
  const ColSumJob job{colsum, colsum_src, rows, cols};
  return gemm_rowmajor(TA == CCT_NO_TRANS, TB == CCT_TRANS, M, N, K, alpha, A, lda, B, ldb, beta, C, N,
                       EPI_ALPHA_BETA, 0, nullptr, 0, nullptr, &job);
}

extern "C" int cct_hip_sgemm_new_bias(int TA, int TB, int M, int N, int K, float alpha, const float *A,
                                      const float *B, float beta, float *C, const float *col_bias, int relu) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE((TA == CCT_NO_TRANS || TA == CCT_TRANS) && (TB == CCT_NO_TRANS || TB == CCT_TRANS),
              "sgemm_new_bias: bad transpose flags %d %d", TA, TB);
  CCT_REQUIRE(M >= 0 && N >= 0 && K >= 0, "sgemm_new_bias: negative dimension");
  if (M == 0 || N == 0) return 0;
  CCT_REQUIRE(A && B && C, "sgemm_new_bias: null matrix");
  const int lda = (TA == CCT_NO_TRANS) ? K : M, ldb = (TB == CCT_NO_TRANS) ? N : K;
  return gemm_rowmajor(TA == CCT_NO_TRANS, TB == CCT_TRANS, M, N, K, alpha, A, lda, B, ldb, beta, C, N,
                       EPI_ALPHA_BETA, 0, nullptr, relu != 0, col_bias);
}

extern "C" int cct_hip_sgemm_conv_forward(int o, int batch, int fmap, int K, const float *model,
                                          const float *lowered, const float *bias, float *out, int relu) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(o > 0 && batch > 0 && fmap > 0 && K > 0, "sgemm_conv_forward: non-positive dimension");
  CCT_REQUIRE(model && lowered && out, "sgemm_conv_forward: null matrix");
  CCT_REQUIRE((size_t)batch * fmap < (1ull << 31), "sgemm_conv_forward: too many output positions");
  return gemm_rowmajor(true, true, o, batch * fmap, K, 1.0f, model, K, lowered, K, 0.0f, out, batch * fmap,
                       EPI_CONV_FORWARD, fmap, bias, relu != 0);
}

// ---- 1 x 1 convolution (stride 1, no padding): products on the tensors as they lie ---------------------------
// A 1 x 1 filter needs no lowering: with `plane` = n*n pixels per map, image i of the input IS the d x plane
// matrix of its lowered form.  Forward and data gradient are one product over the pixels of all images (or one per
// image, all in one launch: conv1x1_across_images below); the weight gradient is one product summed over the
// images.
static bool conv1x1_dims_ok(int batch, int depth, int plane, int num_outputs) {
  return batch > 0 && depth > 0 && plane > 0 && num_outputs > 0 && (double)depth * plane < 2147483648.0 &&
         (double)num_outputs * plane < 2147483648.0 && (double)depth * num_outputs < 2147483648.0;
}

// Forward and data gradient as ONE product whose columns run over the pixels of all images: no tile is padded per
// image (a 14 x 14 map fills 196 of 256 tile columns otherwise).  Measured over 107 layers, against one product
// per image: 13 % less time on 14 x 14 maps, 9 % on 13 x 13, 5 % on 27 x 27 and 28 x 28, 2 % on 7 x 7 (planes
// that are not a multiple of four floats pay for their straddling vectors with scalar loads), 1 % more on
// 56 x 56, where the padding is small -- so planes above 2048 pixels, and planes shorter than one vector, keep one
// product per image.  The tuning knob conv1x1_per_image pins either (1: per image, 2: across images).
static bool conv1x1_across_images(int batch, int plane) {
  if (plane < 4 || (double)batch * plane >= 2147483648.0) return false;
  const int knob = tuning().conv1x1_per_image;
  return knob == 2 || (knob == 0 && plane <= 2048);
}

extern "C" int cct_hip_conv1x1_supported(int batch, int depth, int n, int k, int stride, int padding,
                                         int num_outputs) {
  return k == 1 && stride == 1 && padding == 0 && n > 0 && (double)n * n < 2147483648.0 &&
                 conv1x1_dims_ok(batch, depth, n * n, num_outputs)
             ? 1
             : 0;
}

extern "C" int cct_hip_conv1x1_forward(float *output, const float *input, const float *model, const float *bias,
                                       int batch, int depth, int plane, int num_outputs, int relu) {
  CCT_ENSURE_INIT();
  if (batch == 0) return 0;
  CCT_REQUIRE(conv1x1_dims_ok(batch, depth, plane, num_outputs), "conv1x1_forward: bad dimensions");
  CCT_REQUIRE(output && input && model, "conv1x1_forward: null argument");
  // out_i [o x plane] = model [o x d] * in_i [d x plane] + bias per row
  if (conv1x1_across_images(batch, plane)) {
    // one product over the pixels of all images: [o x batch*plane], stored image by image
    const GemmBatch gb{3, batch, 0, (size_t)depth * plane, 0};
    return gemm_rowmajor(true, false, num_outputs, batch * plane, depth, 1.0f, model, depth, input, plane, 0.0f,
                         output, batch * plane, EPI_CONV_FORWARD, plane, bias, relu != 0, nullptr, nullptr, &gb);
  }
  const GemmBatch gb{1, batch, 0, (size_t)depth * plane, (size_t)num_outputs * plane};
  return gemm_rowmajor(true, false, num_outputs, plane, depth, 1.0f, model, depth, input, plane, 0.0f, output, plane,
                       EPI_CONV_FORWARD, plane, bias, relu != 0, nullptr, nullptr, &gb);
}

extern "C" int cct_hip_conv1x1_backward_data(float *input_grad, const float *output_grad, const float *model,
                                             int batch, int depth, int plane, int num_outputs) {
  CCT_ENSURE_INIT();
  if (batch == 0) return 0;
  CCT_REQUIRE(conv1x1_dims_ok(batch, depth, plane, num_outputs), "conv1x1_backward_data: bad dimensions");
  CCT_REQUIRE(input_grad && output_grad && model, "conv1x1_backward_data: null argument");
  // din_i [d x plane] = model^T [d x o] * dout_i [o x plane]
  if (conv1x1_across_images(batch, plane)) {
    const GemmBatch gb{3, batch, 0, (size_t)num_outputs * plane, 0};
    return gemm_rowmajor(false, false, depth, batch * plane, num_outputs, 1.0f, model, depth, output_grad, plane, 0.0f,
                         input_grad, batch * plane, EPI_CONV_FORWARD, plane, nullptr, 0, nullptr, nullptr, &gb);
  }
  const GemmBatch gb{1, batch, 0, (size_t)num_outputs * plane, (size_t)depth * plane};
  return gemm_rowmajor(false, false, depth, plane, num_outputs, 1.0f, model, depth, output_grad, plane, 0.0f,
                       input_grad, plane, EPI_ALPHA_BETA, 0, nullptr, 0, nullptr, nullptr, &gb);
}

extern "C" int cct_hip_conv1x1_backward_weights(float *model_grad, float *bias_grad, const float *output_grad,
                                                const float *input, int batch, int depth, int plane,
                                                int num_outputs) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(batch >= 0 && conv1x1_dims_ok(batch > 0 ? batch : 1, depth, plane, num_outputs),
              "conv1x1_backward_weights: bad dimensions");
  CCT_REQUIRE(model_grad && (batch == 0 || (output_grad && input)), "conv1x1_backward_weights: null argument");
  if (batch == 0) {
    if (int rc = cct_hip_memset(model_grad, 0, (size_t)num_outputs * depth * sizeof(float))) return rc;
    return bias_grad ? cct_hip_memset(bias_grad, 0, (size_t)num_outputs * sizeof(float)) : 0;
  }
  // dW [o x d] = sum_i dout_i [o x plane] * in_i^T [plane x d]
  const GemmBatch gb{2, batch, (size_t)num_outputs * plane, (size_t)depth * plane, 0};
  if (int rc = gemm_rowmajor(true, true, num_outputs, depth, plane, 1.0f, output_grad, plane, input, plane, 0.0f,
                             model_grad, depth, EPI_ALPHA_BETA, 0, nullptr, 0, nullptr, nullptr, &gb))
    return rc;
  return bias_grad ? cct_hip_backward_bias(bias_grad, output_grad, plane, num_outputs, batch) : 0;
}
