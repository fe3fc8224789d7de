// Type-1 lowering (im2col) for gfx950, whole batch per launch.
//
//   dst[(bi*m*m + r*m + c) * k*k*d + dd*k*k + kr*k + kc] = src[bi][dd][r*s-p+kr][c*s-p+kc]  (0 outside)
//
// One workgroup owns (image bi, band of RB output rows, slab of DS input channels).  It stages
// the zero-padded input window of that band in LDS with coalesced row reads, then streams out
// the lowered rows with 16-byte stores: consecutive lanes write consecutive addresses of one lowered
// row, each lowered element is written exactly once, padding zeros come from the LDS tile so the store
// loop has no bounds tests.  The per-row-position LDS offsets (the (dd,kr,kc) decomposition)
// are tabulated once per workgroup.
//
// HBM traffic per launch: reads b*d*n*n*4 (plus band halo re-reads, served by L2), writes
// b*m*m*k*k*d*4.  Bound: HBM write bandwidth.
#include "cct_common.h"

namespace cct {

struct LowerParams {
  int n, d, k, s, p, b, m;
  int RB;      // output rows per band
  int DS;      // channels per slab
  int TH, TW;  // staged tile rows / cols per channel
  int seglen;  // DS*k*k floats written per output position by one workgroup
  int rowlen;  // k*k*d
  int nbands, nslabs;
  uint32_t nblocks;
  int chunk_full;  // staged floats per channel for an interior band: ((RB-1)*s + k) * n
  int flat;    // 1: whole rows (one slab) of a length that is not a multiple of 4: flat aligned stores
  FastDiv div_kk, div_k, div_seg, div_n, div_chunk, div_m;
};

constexpr int LOWER_MAX_THREADS = 512;  // block size is chosen per launch (multiple of 64)

// dynamic LDS: [DS*TH*TW floats tile][seglen uint16 offsets]
typedef float lower_f4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float lower_f4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(LOWER_MAX_THREADS) void lower_kernel(float *__restrict__ dst,
                                                              const float *__restrict__ src,
                                                              const LowerParams P) {
  extern __shared__ float lds[];
  const int tile_elems = P.DS * P.TH * P.TW;
  float *tile = lds;
  // the table starts on the next 16-byte boundary so that the float4 clear of the tile cannot touch it
  uint16_t *offs = reinterpret_cast<uint16_t *>(lds + ((tile_elems + 3) & ~3));

  // logical block id -> (bi, band, slab); bands of one image stay on one XCD
  uint32_t id = xcd_remap(blockIdx.x, P.nblocks);
  const int slab = id % P.nslabs;
  id /= P.nslabs;
  const int band = id % P.nbands;
  const int bi = id / P.nbands;

  const int tid = threadIdx.x;
  const int T = blockDim.x;
  const int r0 = band * P.RB;
  const int rb = min(P.RB, P.m - r0);
  const int dd0 = slab * P.DS;
  const int ds = min(P.DS, P.d - dd0);
  const int seg = ds * P.k * P.k;

  // (1) offset table: j = dl*k*k + kr*k + kc  ->  (dl*TH + kr)*TW + kc
  for (int j = tid; j < seg; j += T) {
    const uint32_t dl = fdiv(j, P.div_kk);
    const uint32_t rem = j - dl * P.k * P.k;
    const uint32_t kr = fdiv(rem, P.div_k);
    const uint32_t kc = rem - kr * P.k;
    offs[j] = (uint16_t)((dl * P.TH + kr) * P.TW + kc);
  }

  // (2) stage the padded window: tile[dl][ty][tx] = src[bi][dd0+dl][r0*s-p+ty][-p+tx].
  // The tile is cleared first (that is the zero padding); then the in-image rows of every channel,
  // which are one contiguous run of nrows*n floats in HBM, are copied with eight independent
  // loads in flight per lane.
  {
    const int nz4 = (tile_elems + 3) >> 2;
    float4 *t4 = reinterpret_cast<float4 *>(tile);
    for (int e = tid; e < nz4; e += T) t4[e] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  __syncthreads();
  {
    const int y0 = r0 * P.s - P.p;
    const int th_used = (rb - 1) * P.s + P.k;
    const int ylo = max(y0, 0), yhi = min(y0 + th_used, P.n);
    const int chunk = (yhi - ylo) * P.n;
    const int total = ds * chunk;
    const int nn = P.n * P.n;
    const float *img = src + ((size_t)bi * P.d + dd0) * nn + ylo * P.n;
    const int trow0 = ylo - y0;
    const bool fast = (chunk == P.chunk_full);
    for (int base = 0; base < total; base += T * 8) {
      float v[8];
      int dst_i[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int e = base + j * T + tid;
        const bool ok = e < total;
        const uint32_t ec = ok ? e : 0;
        const uint32_t dl = fast ? fdiv(ec, P.div_chunk) : ec / (uint32_t)chunk;
        const uint32_t i = ec - dl * chunk;
        const uint32_t row = fdiv(i, P.div_n);
        const uint32_t x = i - row * P.n;
        v[j] = img[(size_t)dl * nn + i];
        // columns past the last window (strided layers) have no place in the tile
        dst_i[j] = (ok && (int)x + P.p < P.TW) ? (int)((dl * P.TH + trow0 + row) * P.TW + P.p + x) : -1;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (dst_i[j] >= 0) tile[dst_i[j]] = v[j];
    }
  }
  __syncthreads();

  // (3) stream the lowered rows.
  if (P.flat) {
    // Whole rows whose length is not a multiple of four floats: the band's output -- rb*m lowered
    // rows -- is one contiguous range of HBM, written as a flat stream of 16-byte stores on 16-byte
    // boundaries, consecutive lanes at consecutive addresses (a quad may end one lowered row and
    // begin the next); the up to three floats before the first boundary and after the last go out
    // singly.  Stores that straddle the boundaries (a lane per quad of a row, as below) measured
    // 20 % slower on rows of 363 floats.
    float *ob = dst + ((size_t)bi * P.m + r0) * P.m * P.rowlen;
    const int L = rb * P.m * P.rowlen;
    const int head = min((int)((4 - ((reinterpret_cast<uintptr_t>(ob) >> 2) & 3)) & 3), L);
    const int nq = (L - head) >> 2;
    // tile index of the flat element at row position rp = rl*m + c, column j of the lowered row
    auto tix = [&](int rp, int j) -> int {
      const int rl = P.RB > 1 ? (int)fdiv((uint32_t)rp, P.div_m) : 0;
      return (rl * P.TW + (rp - rl * P.m)) * P.s + offs[j];
    };
    const uint32_t step = 4u * T;
    const int drp = (int)fdiv(step, P.div_seg), dj = (int)(step - (uint32_t)drp * P.rowlen);
    int rp = (int)fdiv((uint32_t)(head + 4 * tid), P.div_seg), j = head + 4 * tid - rp * P.rowlen;
#pragma unroll 2
    for (int q = tid; q < nq; q += T) {
      float w[4];
      if (j + 3 < P.rowlen) {
        const int rl = P.RB > 1 ? (int)fdiv((uint32_t)rp, P.div_m) : 0;
        const float *t = tile + (rl * P.TW + (rp - rl * P.m)) * P.s;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = t[offs[j + i]];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ji = j + i, wrap = ji >= P.rowlen;
          w[i] = tile[tix(rp + wrap, ji - (wrap ? P.rowlen : 0))];
        }
      }
      *reinterpret_cast<lower_f4 *>(ob + head + 4 * (size_t)q) = lower_f4{w[0], w[1], w[2], w[3]};
      rp += drp; j += dj;
      if (j >= P.rowlen) { j -= P.rowlen; ++rp; }
    }
    const int ntail = L - head - 4 * nq;
    if (tid < head + ntail) {
      const int f = tid < head ? tid : head + 4 * nq + (tid - head);
      const int rpf = (int)fdiv((uint32_t)f, P.div_seg);
      ob[f] = tile[tix(rpf, f - rpf * P.rowlen)];
    }
    return;
  }
  // Otherwise a lane owns a unit -- 4 consecutive positions of a lowered row (one 16-byte store;
  // dword alignment is all such a store needs) or one of the seg % 4 positions left over -- and a
  // group of output columns, and walks over the band.  Short rows (few units) are spread over
  // several column groups so that the whole workgroup stores.
  float *out_band = dst + ((size_t)bi * P.m + r0) * P.m * P.rowlen + (size_t)dd0 * P.k * P.k;
  const int nq = seg >> 2, units = nq + (seg & 3);
  const int groups = units < T ? min(T / units, P.m) : 1;
  const int cpg = (P.m + groups - 1) / groups;
  for (int wi = tid; wi < units * groups; wi += T) {
    const int cg = groups > 1 ? wi / units : 0, u = wi - cg * units;
    const int c_lo = cg * cpg, c_hi = min(P.m, c_lo + cpg);
    if (u < nq) {
      const int o0 = offs[4 * u], o1 = offs[4 * u + 1], o2 = offs[4 * u + 2], o3 = offs[4 * u + 3];
      float *outq = out_band + 4 * u;
      for (int rl = 0; rl < rb; ++rl) {
        const float *trow = tile + rl * P.s * P.TW;
        float *orow = outq + (size_t)rl * P.m * P.rowlen;
#pragma unroll 4
        for (int c = c_lo; c < c_hi; ++c) {
          const float *t = trow + c * P.s;
          const lower_f4u v = {t[o0], t[o1], t[o2], t[o3]};
          *reinterpret_cast<lower_f4u *>(orow + (size_t)c * P.rowlen) = v;
        }
      }
    } else {
      const int j = 4 * nq + (u - nq), o = offs[j];
      for (int rl = 0; rl < rb; ++rl) {
        const float *trow = tile + rl * P.s * P.TW;
        float *orow = out_band + j + (size_t)rl * P.m * P.rowlen;
        for (int c = c_lo; c < c_hi; ++c) orow[(size_t)c * P.rowlen] = trow[c * P.s + o];
      }
    }
  }
}

}  // namespace cct

using namespace cct;

extern "C" int cct_hip_lower_cube(float *dst, const float *src, const cct_pmap_helper *a) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dst && src && a, "lower_cube: null argument");
  // same preconditions as CPUDriver::lower_cube (src/sched/DeviceDriver_CPU.cpp:137-140)
  CCT_REQUIRE(a->sR == a->sC, "lower_cube: input must be square (sR=%zu sC=%zu)", a->sR, a->sC);
  CCT_REQUIRE(a->kR == a->kC, "lower_cube: kernel must be square (kR=%zu kC=%zu)", a->kR, a->kC);
  CCT_REQUIRE(a->stride >= 1, "lower_cube: stride must be >= 1");
  CCT_REQUIRE(a->kR >= 1 && a->sR + 2 * a->padding >= a->kR, "lower_cube: kernel larger than padded input");
  if (a->sB == 0 || a->sD == 0) return 0;

  LowerParams P;
  P.n = (int)a->sR; P.d = (int)a->sD; P.k = (int)a->kR; P.s = (int)a->stride;
  P.p = (int)a->padding; P.b = (int)a->sB;
  P.m = (P.n + 2 * P.p - P.k) / P.s + 1;
  P.rowlen = P.k * P.k * P.d;
  const size_t out_elems = (size_t)P.b * P.m * P.m * P.rowlen;
  CCT_REQUIRE((size_t)P.b * P.d * P.n * P.n < (1ull << 31) && out_elems / P.rowlen < (1ull << 31),
              "lower_cube: tensor too large for 31-bit position arithmetic");

  // Tile sizing: keep the staged window within 78 KB so two workgroups share a CU's 160 KB LDS,
  // keep the uint16 offset table valid (< 65536 tile elements), prefer whole rows (DS = d).
  const size_t lds_budget = 78 * 1024;
  P.TW = (P.m - 1) * P.s + P.k;
  P.RB = 1;
  P.DS = P.d;
  auto lds_need = [&](int RB, int DS) {
    const size_t th = (size_t)(RB - 1) * P.s + P.k;
    return ((((size_t)DS * th * P.TW) + 3) & ~(size_t)3) * 4 + (((size_t)DS * P.k * P.k * 2 + 3) & ~(size_t)3);
  };
  while (P.DS > 1 && (lds_need(1, P.DS) > lds_budget || (size_t)P.DS * P.k * P.TW >= 65536))
    P.DS = (P.DS + 1) / 2;
  CCT_REQUIRE(lds_need(1, P.DS) <= 150 * 1024 && (size_t)P.DS * P.k * P.TW < 65536,
              "lower_cube: one channel window (%d x %d floats) does not fit in LDS", P.k, P.TW);
  // A one-row band re-reads k/s times the input, but the input is small against the lowered output and
  // L2 serves the re-reads: for stride 1 one-row bands (more, smaller workgroups in flight) measured 5 %
  // faster than wider ones.  Strided layers widen the band while it fits.
  if (P.s > 1 && P.s < P.k) {
    while (P.RB < P.m && P.RB < 8 && lds_need(P.RB * 2, P.DS) <= lds_budget &&
           (size_t)P.DS * ((size_t)(P.RB * 2 - 1) * P.s + P.k) * P.TW < 65536 &&
           (size_t)P.b * ((P.m + P.RB * 2 - 1) / (P.RB * 2)) >= 2048)
      P.RB *= 2;
  }
  P.TH = (P.RB - 1) * P.s + P.k;
  P.seglen = P.DS * P.k * P.k;
  P.nbands = (P.m + P.RB - 1) / P.RB;
  P.nslabs = (P.d + P.DS - 1) / P.DS;
  const size_t nblocks = (size_t)P.b * P.nbands * P.nslabs;
  CCT_REQUIRE(nblocks < (1ull << 31), "lower_cube: too many workgroups");
  P.nblocks = (uint32_t)nblocks;
  P.chunk_full = P.TH * P.n;
  P.div_kk = make_fastdiv(P.k * P.k);
  P.div_k = make_fastdiv(P.k);
  P.div_seg = make_fastdiv(P.seglen);
  P.div_n = make_fastdiv(P.n);
  P.div_m = make_fastdiv(P.m);
  P.flat = P.nslabs == 1 && (P.rowlen & 3) != 0 && P.rowlen >= 4;  // a quad then spans at most two lowered rows
  P.div_chunk = make_fastdiv(P.chunk_full);

  const size_t lds_bytes = lds_need(P.RB, P.DS);
  // block size (a multiple of 64).  Flat stores balance any size: the largest workgroup unless the
  // band is small.  Otherwise close to a whole number of (unit, column group) work items; rows
  // with many units take the largest size (measured faster than the size that wastes the fewest
  // lanes of the last pass: more stores in flight per compute unit).
  const long units = P.seglen / 4 + P.seglen % 4;
  int threads = LOWER_MAX_THREADS;
  if (P.flat) {
    const long quads = (long)P.RB * P.m * P.rowlen / 4;
    if (quads < 4 * LOWER_MAX_THREADS) threads = (int)((quads / 4 + 63) / 64 * 64);
    if (threads < 128) threads = 128;
  } else if (units < LOWER_MAX_THREADS) {
    // several column groups per workgroup: as many lanes as the groups use, rounded up to wavefronts
    const long groups = LOWER_MAX_THREADS / units < P.m ? LOWER_MAX_THREADS / units : P.m;
    threads = (int)((units * groups + 63) / 64 * 64);
    if (threads > LOWER_MAX_THREADS) threads = LOWER_MAX_THREADS;
    if (threads < 128) threads = 128;
  }
  hipStream_t st = ctx().stream;
  static LdsGrant grant;
  if (int rc = grant_dynamic_lds((const void *)lower_kernel, lds_bytes, grant)) return rc;
  hipLaunchKernelGGL(lower_kernel, dim3(P.nblocks), dim3(threads), lds_bytes, st, dst, src, P);
  CCT_LAUNCH_CHECK();
  note_kernel("lower_kernel threads=%d%s", threads, P.flat ? " flat" : "");
  return 0;
}
