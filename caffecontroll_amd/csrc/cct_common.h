// Shared internals of the gfx950 driver library: process state, error plumbing, small
// device helpers.  Not part of the public ABI (that is include/cct_hip.h).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "../../include/cct_hip.h"

namespace cct {

struct Context {
  int device = -1;
  int compute_units = 0;
  hipStream_t stream = nullptr;
  // grow-only device workspace for split-K partial sums
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  // zero-initialised arrival counters for reductions finished by the last workgroup (self-resetting)
  unsigned int *counters = nullptr;
  // dropout generator state: seed and number of rand_uint_initialize calls so far
  uint64_t rng_seed = 0;
  uint64_t rng_calls = 0;
};

// Tuning overrides, for experiments and for tests that pin a kernel instance.  Read ONCE from the
// environment when the library initialises (CCT_HIP_DIRECT_TILE, _DIRECT_WAVES, _DIRECT_TB,
// _DIRECT_NOSPEC, _DIRECT_SPLITS, _DIRECT_ALDS, _DIRECT_WGRAD_ROWS, _STRIDED_WGRAD, _POOL_PLANE, _GEMM_NT, _GEMM_TILE, _GEMM_NODMA), changed afterwards only through
// cct_hip_set_tuning(); the launch paths read this struct, never the environment.
struct Tuning {
  int direct_tile = 0;    // "<map blocks><pixel blocks>" of conv_direct_kernel, 0 = model's choice
  int direct_waves = 0;   // wavefronts of the weight-gradient workgroup (4..8), 0 = model's choice
  int direct_tb = 0;      // column blocks of the weight-gradient tile (1..6), 0 = model's choice
  int direct_nospec = 0;  // 1: never take the shape-specialised weight-gradient instances
  int direct_splits = 0;  // step ranges of the weight-gradient launch (its partial sums), 0 = model's choice
  int direct_alds = 0;    // specialised weight-gradient instances: 1 = dout rows through LDS, 2 = never, 0 = model's choice
  int conv1x1_per_image = 0;  // 1 x 1 layers, forward and data gradient: 1 = one product per image, 2 = one product over the pixels of all images, 0 = by plane size
  int direct_wgrad_rows = 0;  // stride-1 weight gradient: 1 = image-pair kernels wherever they apply, 2 = one image per step always, 0 = model's choice
  int strided_wgrad = 0;  // strided weight-gradient tile: row pieces * 1000 + column blocks * 100 + column groups * 10 + row blocks, 0 = model's choice
  int pool_plane = 0;     // 1: plane-tiled pooling kernels at any size
  int gemm_nt = 0;        // 1: non-temporal stores in the GEMM epilogue
  int gemm_tile = -1;     // index of the GEMM tile shape, -1 = model's choice
  int gemm_nodma = 0;     // 1: GEMM operand tiles always staged through registers
};
Tuning &tuning();

Context &ctx();
int ensure_init();
int set_error(int code, const char *fmt, ...);
int get_workspace(size_t bytes, void **out);
constexpr int kMaxCounters = 16384;
int get_counters(unsigned int **out);
// A launch that used the arrival counters failed or was refused: they are cleared before their next use.
void mark_counters_dirty();

// Kernels that need more than 64 KB of dynamic LDS must be granted it once per device; `st` (one
// static object per kernel instance) remembers the grant so that later launches skip the call.
struct LdsGrant {
  int device = -1;
  size_t bytes = 0;
};
int grant_dynamic_lds(const void *kernel, size_t bytes, LdsGrant &st);

// Records the instance the launch path chose for the product kernel it just enqueued (template
// arguments in the order a kernel trace prints them, plus launch-time choices such as the split
// count); cct_hip_last_kernel() returns the most recent record.
void note_kernel(const char *fmt, ...);

#define CCT_HIP_CHECK(expr)                                                                    \
  do {                                                                                         \
    hipError_t _e = (expr);                                                                    \
    if (_e != hipSuccess)                                                                      \
      return ::cct::set_error((int)_e, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),  \
                              __FILE__, __LINE__);                                             \
  } while (0)

#define CCT_REQUIRE(cond, ...)                                          \
  do {                                                                  \
    if (!(cond)) return ::cct::set_error(CCT_HIP_EINVAL, __VA_ARGS__);  \
  } while (0)

#define CCT_ENSURE_INIT()               \
  do {                                  \
    int _rc = ::cct::ensure_init();     \
    if (_rc) return _rc;                \
  } while (0)

// Checks the launch that was just enqueued.
#define CCT_LAUNCH_CHECK() CCT_HIP_CHECK(hipGetLastError())

// Division of 31-bit numerators by a launch-time constant: q = mulhi(n, mul) >> shift.
// Exact for every 0 <= n < 2^31 (mul = ceil(2^(31+l)/d), l = ceil(log2 d)); d == 1 is flagged.
struct FastDiv {
  uint32_t mul;
  uint32_t shift;
  uint32_t div;
};

inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.div = d;
  if (d <= 1) {
    f.mul = 0;
    f.shift = 0;
    return f;
  }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;
  const unsigned __int128 num = (unsigned __int128)1 << (31 + l);
  f.mul = (uint32_t)((num + d - 1) / d);
  f.shift = l - 1;
  return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f) {
  return f.div <= 1 ? n : (__umulhi(n, f.mul) >> f.shift);
}

// XCD-aware block renumbering.  Hardware hands consecutive workgroup ids to the 8 XCDs round
// robin; this maps the id so that each XCD walks one contiguous range of logical tiles, which
// keeps tiles that share input on the same L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t id, uint32_t total) {
  const uint32_t nx = 8;
  const uint32_t q = total / nx, r = total % nx;
  const uint32_t x = id % nx, i = id / nx;
  const uint32_t base = (x < r) ? x * (q + 1) : r * (q + 1) + (x - r) * q;
  return base + i;
}

}  // namespace cct
