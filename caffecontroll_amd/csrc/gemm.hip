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
#include "cct_common.h"

namespace cct {

typedef float v16f __attribute__((ext_vector_type(16)));

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
  int tiles_m, tiles_n;
  uint32_t ntiles;
  int a_vec, b_vec;  // operand allows aligned 16-byte global loads
};

__device__ __forceinline__ float4 ldg4(const float *__restrict__ base, int major, int minor,
                                       int major_lim, int minor_lim, int ld, int vec) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (major < major_lim) {
    const float *p = base + (size_t)major * ld + minor;
    if (vec && minor + 3 < minor_lim) {
      v = *reinterpret_cast<const float4 *>(p);
    } else {
      if (minor + 0 < minor_lim) v.x = p[0];
      if (minor + 1 < minor_lim) v.y = p[1];
      if (minor + 2 < minor_lim) v.z = p[2];
      if (minor + 3 < minor_lim) v.w = p[3];
    }
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
  static_assert((BM * BK / 4) % THREADS == 0 && (BN * BK / 4) % THREADS == 0, "loader coverage");
};

template <class T, bool KC, int ROWS>
struct OperandLayout {
  // floats per LDS stage
  static constexpr int SIZE = KC ? ROWS * (T::BK + T::PK) : T::BK * (ROWS + T::PR);
  static constexpr int NV = ROWS * T::BK / 4 / T::THREADS;  // float4 per lane per stage
};

// global -> registers for one operand tile (rows x BK) starting at (row0, k0)
template <class T, bool KC, int ROWS>
__device__ __forceinline__ void load_tile(float4 *__restrict__ r,
                                          const float *__restrict__ g, int ld, int row0, int k0,
                                          int row_lim, int k_lim, int vec, int tid) {
  constexpr int NV = OperandLayout<T, KC, ROWS>::NV;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int f = tid + i * T::THREADS;
    if (KC) {
      const int row = f / (T::BK / 4), kq = f % (T::BK / 4);
      r[i] = ldg4(g, row0 + row, k0 + kq * 4, row_lim, k_lim, ld, vec);
    } else {
      const int kk = f / (ROWS / 4), rq = f % (ROWS / 4);
      r[i] = ldg4(g, k0 + kk, row0 + rq * 4, k_lim, row_lim, ld, vec);
    }
  }
}

template <class T, bool KC, int ROWS>
__device__ __forceinline__ void store_tile(float *__restrict__ lds, const float4 *__restrict__ r,
                                           int tid) {
  constexpr int NV = OperandLayout<T, KC, ROWS>::NV;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int f = tid + i * T::THREADS;
    if (KC) {
      const int row = f / (T::BK / 4), kq = f % (T::BK / 4);
      *reinterpret_cast<float4 *>(lds + row * (T::BK + T::PK) + kq * 4) = r[i];
    } else {
      const int kk = f / (ROWS / 4), rq = f % (ROWS / 4);
      *reinterpret_cast<float4 *>(lds + kk * (ROWS + T::PR) + rq * 4) = r[i];
    }
  }
}

// fragments of k-group kg for NT 32-row tiles starting at row0: f[t][i], i = MFMA index in group
template <class T, bool KC, int ROWS, int NT>
__device__ __forceinline__ void load_frags(float (&f)[NT][4], const float *__restrict__ lds,
                                           int row0, int kg, int lane) {
  const int r = lane & 31, h = lane >> 5;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (KC) {
      const float4 v = *reinterpret_cast<const float4 *>(lds + (row0 + t * 32 + r) * (T::BK + T::PK) +
                                                         kg * 8 + h * 4);
      f[t][0] = v.x; f[t][1] = v.y; f[t][2] = v.z; f[t][3] = v.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        f[t][i] = lds[(kg * 8 + h * 4 + i) * (ROWS + T::PR) + row0 + t * 32 + r];
    }
  }
}

template <class T, bool A_KC, bool B_KC>
__global__ __launch_bounds__(T::THREADS, 2) void gemm_kernel(const GemmArgs g) {
  using LA = OperandLayout<T, A_KC, T::BM>;
  using LB = OperandLayout<T, B_KC, T::BN>;
  __shared__ __attribute__((aligned(16))) float smem[2 * (LA::SIZE + LB::SIZE)];
  constexpr int STAGE = LA::SIZE + LB::SIZE;  // stage s: A at smem + s*STAGE, B right after it

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / T::WGN) * T::WM, wn0 = (wave % T::WGN) * T::WN;

  // tile id: the dimension with fewer tiles runs fastest so that neighbouring workgroups on one
  // XCD share the larger operand tile in L2
  const uint32_t id = xcd_remap(blockIdx.x, g.ntiles);
  int tm, tn;
  if (g.tiles_m <= g.tiles_n) {
    tm = id % g.tiles_m; tn = id / g.tiles_m;
  } else {
    tn = id % g.tiles_n; tm = id / g.tiles_n;
  }
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int kbeg = blockIdx.y * g.kchunk;
  const int kend = min(g.K, kbeg + g.kchunk);
  const int nk = (kend - kbeg + T::BK - 1) / T::BK;

  v16f acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  float4 ra[LA::NV], rb[LB::NV];
  if (nk > 0) {
    load_tile<T, A_KC, T::BM>(ra, g.A, g.lda, m0, kbeg, g.M, kend, g.a_vec, tid);
    load_tile<T, B_KC, T::BN>(rb, g.B, g.ldb, n0, kbeg, g.N, kend, g.b_vec, tid);
    store_tile<T, A_KC, T::BM>(smem, ra, tid);
    store_tile<T, B_KC, T::BN>(smem + LA::SIZE, rb, tid);
  }
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = (kt + 1 < nk);
    if (more) {
      const int k0 = kbeg + (kt + 1) * T::BK;
      load_tile<T, A_KC, T::BM>(ra, g.A, g.lda, m0, k0, g.M, kend, g.a_vec, tid);
      load_tile<T, B_KC, T::BN>(rb, g.B, g.ldb, n0, k0, g.N, kend, g.b_vec, tid);
    }
    const float *as = smem + cur * STAGE;
    const float *bs = as + LA::SIZE;
#pragma unroll
    for (int kg = 0; kg < T::BK / 8; ++kg) {
      float fa[T::TM][4], fb[T::TN][4];
      load_frags<T, A_KC, T::BM, T::TM>(fa, as, wm0, kg, lane);
      load_frags<T, B_KC, T::BN, T::TN>(fb, bs, wn0, kg, lane);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int a = 0; a < T::TM; ++a)
#pragma unroll
          for (int b = 0; b < T::TN; ++b)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a][i], fb[b][i], acc[a][b], 0, 0, 0);
    }
    if (more) {
      store_tile<T, A_KC, T::BM>(smem + (cur ^ 1) * STAGE, ra, tid);
      store_tile<T, B_KC, T::BN>(smem + (cur ^ 1) * STAGE + LA::SIZE, rb, tid);
    }
    __syncthreads();
  }

  // epilogue: accumulator register v of lane (r,h) is C[8*(v/4) + 4*h + v%4][r] of its 32x32 tile
  const int r = lane & 31, h = lane >> 5;
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
          float *c = g.C + (size_t)row * g.ldc + col_off;
          *c = (g.beta == 0.0f) ? g.alpha * x : g.alpha * x + g.beta * (*c);
        } else if (g.epi == EPI_SPLITK_PARTIAL) {
          g.ws[((size_t)blockIdx.y * g.M + row) * g.N + col_off] = x;
        } else {
          g.C[(size_t)row * g.fmap + col_off] = g.bias ? x + g.bias[row] : x;
        }
      }
    }
  }
}

// C = alpha * sum_z ws[z] + beta * C, z ascending (fixed order)
__global__ __launch_bounds__(256) void splitk_reduce_kernel(float *__restrict__ C,
                                                            const float *__restrict__ ws, int M, int N,
                                                            int ldc, int splits, float alpha, float beta,
                                                            FastDiv div_n) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= (uint32_t)M * N) return;
  const uint32_t row = fdiv(e, div_n);
  const uint32_t col = e - row * N;
  float s = 0.0f;
  const size_t mn = (size_t)M * N;
  for (int z = 0; z < splits; ++z) s += ws[(size_t)z * mn + e];
  float *c = C + (size_t)row * ldc + col;
  *c = (beta == 0.0f) ? alpha * s : alpha * s + beta * (*c);
}

typedef Tile<256, 128, 16, 2, 2> TileL;
typedef Tile<128, 128, 16, 2, 2> TileM;
typedef Tile<64, 64, 16, 2, 2> TileS;

template <class T>
static int launch_cfg(GemmArgs &g, bool a_kc, bool b_kc, int splits, hipStream_t st) {
  g.tiles_m = (g.M + T::BM - 1) / T::BM;
  g.tiles_n = (g.N + T::BN - 1) / T::BN;
  g.ntiles = (uint32_t)g.tiles_m * g.tiles_n;
  dim3 grid(g.ntiles, splits), block(T::THREADS);
  if (a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, true>), grid, block, 0, st, g);
  else if (a_kc && !b_kc) hipLaunchKernelGGL((gemm_kernel<T, true, false>), grid, block, 0, st, g);
  else if (!a_kc && b_kc) hipLaunchKernelGGL((gemm_kernel<T, false, true>), grid, block, 0, st, g);
  else hipLaunchKernelGGL((gemm_kernel<T, false, false>), grid, block, 0, st, g);
  CCT_LAUNCH_CHECK();
  return 0;
}

// Row-major GEMM driver.  a_kc: A(m,k) = A[m*lda + k] (cblas NoTrans); b_kc: B(k,n) = B[n*ldb + k]
// (cblas Trans).
static int gemm_rowmajor(bool a_kc, bool b_kc, int M, int N, int K, float alpha, const float *A, int lda,
                         const float *B, int ldb, float beta, float *C, int ldc, int epi, int fmap,
                         const float *bias) {
  if (M <= 0 || N <= 0) return 0;
  hipStream_t st = ctx().stream;
  GemmArgs g;
  g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.alpha = alpha; g.beta = beta; g.epi = epi; g.fmap = fmap > 0 ? fmap : 1;
  g.div_fmap = make_fastdiv((uint32_t)g.fmap); g.bias = bias; g.ws = nullptr;
  g.a_vec = ((uintptr_t)A % 16 == 0) && (lda % 4 == 0);
  g.b_vec = ((uintptr_t)B % 16 == 0) && (ldb % 4 == 0);
  if (K <= 0) g.K = 0;  // degenerate: C = beta*C through the normal epilogue with zero accumulators

  // tile choice: largest macro tile that still yields at least one workgroup per compute unit
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  auto ntiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  int cfg;  // 0 = L, 1 = M, 2 = S
  if (M > 128 && N >= 128 && (M % 256 == 0 || M > 512)) cfg = 0;
  else if (M > 64 && N > 64) cfg = 1;
  else cfg = 2;
  const int bm = cfg == 0 ? 256 : cfg == 1 ? 128 : 64, bn = cfg == 2 ? 64 : 128, bk = 16;
  const long tiles = ntiles(bm, bn);

  // split-K only for the plain epilogue when the tile grid cannot fill the device
  int splits = 1;
  const long slots = 2L * cus;
  if (epi == EPI_ALPHA_BETA && tiles < cus && K >= 1024) {
    splits = (int)(slots / tiles);
    const int max_splits = K / 256;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
  }
  int kchunk = g.K > 0 ? g.K : bk;
  if (splits > 1) {
    kchunk = (((K + splits - 1) / splits) + bk - 1) / bk * bk;
    splits = (K + kchunk - 1) / kchunk;
  }
  g.kchunk = kchunk;
  if (splits > 1) {
    void *ws = nullptr;
    int rc = get_workspace((size_t)splits * M * N * sizeof(float), &ws);
    if (rc) return rc;
    g.ws = (float *)ws;
    g.epi = EPI_SPLITK_PARTIAL;
  }
  int rc = cfg == 0   ? launch_cfg<TileL>(g, a_kc, b_kc, splits, st)
           : cfg == 1 ? launch_cfg<TileM>(g, a_kc, b_kc, splits, st)
                      : launch_cfg<TileS>(g, a_kc, b_kc, splits, st);
  if (rc) return rc;
  if (splits > 1) {
    CCT_REQUIRE((size_t)M * N < (1ull << 31), "sgemm: split-K result too large");
    const uint32_t blocks = (uint32_t)(((size_t)M * N + 255) / 256);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, st, C, g.ws, M, N, ldc, splits,
                       alpha, beta, make_fastdiv((uint32_t)N));
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

extern "C" int cct_hip_sgemm_conv_forward(int o, int batch, int fmap, int K, const float *model,
                                          const float *lowered, const float *bias, float *out) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(o > 0 && batch > 0 && fmap > 0 && K > 0, "sgemm_conv_forward: non-positive dimension");
  CCT_REQUIRE(model && lowered && out, "sgemm_conv_forward: null matrix");
  CCT_REQUIRE((size_t)batch * fmap < (1ull << 31), "sgemm_conv_forward: too many output positions");
  return gemm_rowmajor(true, true, o, batch * fmap, K, 1.0f, model, K, lowered, K, 0.0f, out, batch * fmap,
                       EPI_CONV_FORWARD, fmap, bias);
}
