// Pieces shared by the direct-convolution kernels (stride 1: direct.hip; strided: strided.hip):
// MFMA vector types and the global -> LDS transfer helpers.
#pragma once
#include "cct_common.h"

namespace cct {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));


// global -> LDS without passing through registers, as buffer loads: the address is
// descriptor base + scalar offset + per-lane 32-bit byte offset, and a lane whose offset is
// kOutOfRange (>= the descriptor's size) fetches nothing and writes zero.  `lds_wave_base` is the
// wave-uniform LDS address that lane 0's data goes to; lane l's 16 (or 4) bytes land 16*l (4*l)
// bytes further on.  The scalar offset does not take part in the range test, so every descriptor
// is given the size 2^31 and the real bounds are kept by the callers' own index logic.
typedef __attribute__((address_space(3))) void lds_void;
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr uint32_t kOutOfRange = 0x80000000u;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)kOutOfRange, 0x00020000);
}
// a descriptor of size zero: every lane is out of range whatever its offset
__device__ __forceinline__ rsrc_t make_rsrc_empty(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0, 0x00020000);
}
__device__ __forceinline__ void lds_dma16(rsrc_t r, uint32_t lane_bytes, uint32_t wave_bytes, float *lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void *)(uintptr_t)lds_wave_base, 16, lane_bytes, wave_bytes, 0, 0);
}
__device__ __forceinline__ void lds_dma4(rsrc_t r, uint32_t lane_bytes, uint32_t wave_bytes, float *lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void *)(uintptr_t)lds_wave_base, 4, lane_bytes, wave_bytes, 0, 0);
}
// all of this wave's global->LDS loads have landed (vmcnt(0); expcnt/lgkmcnt left alone)
__device__ __forceinline__ void lds_dma_wait() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// dst[e] = sum over z of ws[z][e] for e < n, and dst2[e] = sum over z of ws2[z][e] for e < n2 (z ascending):
// the fixed-order reduction of the partial sums the weight-gradient kernels leave in the workspace
// (defined beside the stride-1 kernels).
int reduce_partial_sums(float *dst, const float *ws, uint32_t n, float *dst2, const float *ws2, uint32_t n2,
                        int splits, hipStream_t st);

// Weight (and bias) gradient kernel that stages one output row of ONE image per step (defined beside the strided
// kernels): strided layers, and stride-1 layers whose rows are too long for the image-pair kernels.
bool conv_strided_wgrad_covers(int batch, int d, int n, int ks, int stride, int pad, int o);
int conv_strided_wgrad(float *dw, float *db, const float *dout, const float *src, int batch, int d, int n, int ks,
                       int stride, int pad, int o, size_t src_img_stride, size_t dout_img_stride);

}  // namespace cct
