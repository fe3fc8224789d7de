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

Context &ctx();
int ensure_init();
int set_error(int code, const char *fmt, ...);
int get_workspace(size_t bytes, void **out);
constexpr int kMaxCounters = 16384;
int get_counters(unsigned int **out);

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
