// Column sums of a dense row-major matrix, dst[d] = sum over b of src[b][d] (the bias gradient of an inner-product
// layer, backward_bias_fc: src/sched/DeviceDriver_CPU.cpp:264-286), as the work of ONE 256-lane workgroup on 64
// columns: its four wavefronts sum a quarter of the rows each (ascending, eight loads in flight per lane) and the four
// partial sums are added in a fixed order.  Shared by the kernel of its own and by the launches that carry the sums
// along in spare workgroups, so that a layer's bias gradient is the same bits whichever launch computed it.
#pragma once
#include "cct_common.h"

namespace cct {

// `part`: 4 x 64 floats of LDS; `block`: which 64 columns.  All 256 lanes of the workgroup must call it.
__device__ __forceinline__ void colsum_block(float *__restrict__ dst, const float *__restrict__ src, int D, int B,
                                             uint32_t block, float (*part)[64]) {
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int d = (int)block * 64 + lane;
  const int per = (B + 3) / 4, b0 = q * per, b1 = min(B, b0 + per);
  float s = 0.0f;
  if (d < D) {
    const float *p = src + (size_t)b0 * D + d;
    int b = b0;
    for (; b + 8 <= b1; b += 8, p += (size_t)8 * D) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = p[(size_t)j * D];
#pragma unroll
      for (int j = 0; j < 8; ++j) s += v[j];
    }
    for (; b < b1; ++b, p += D) s += *p;
  }
  part[q][lane] = s;
  __syncthreads();
  if (q == 0 && d < D) dst[d] = ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane];
}

}  // namespace cct
