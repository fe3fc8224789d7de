// GEMM "kernel" object: maps the reference's KernelConfig to (TA, TB, M, N, K, lda, ldb) and
// calls driver->sgemm(CblasRowMajor, ...).  Counterpart of
// Kernel<..., Kernel_GEMM_OpenBlas, KERNELCONFIG, DriverClass>::compute (src/Kernel_impl.hxx:85-170).
#pragma once
#include "LogicalCube.h"

namespace cct {

enum KernelConfig {
  KernelConfig_GEMM_NOTRANS_NOTRANS,
  KernelConfig_GEMM_NOTRANS_TRANS,
  KernelConfig_GEMM_TRANS_NOTRANS,
  KernelConfig_GEMM_NOTRANS_TRANS_NO_DIM_FLIP,
  KernelConfig_GEMM_TRANS_NO_DIM_FLIP_NOTRANS,
  KernelConfig_GEMM_NOTRANS_NOTRANS_DIM_FLIP,
  KernelConfig_GEMM_NOTRANS_DIM_FLIP_NOTRANS
};

template <typename DataType, KernelConfig KERNELCONFIG, typename DriverClass>
class Kernel {
 public:
  typedef LogicalCube<DataType> CubeType;
  const size_t i1R, i1C, i2R, i2C, oR, oC;
  float alpha, beta;

  Kernel(const CubeType *const p_input1_cube, const CubeType *const p_input2_cube,
         const CubeType *const p_output_cube, DriverClass *_p_driver)
      : i1R(p_input1_cube->R), i1C(p_input1_cube->C), i2R(p_input2_cube->R), i2C(p_input2_cube->C),
        oR(p_output_cube->R), oC(p_output_cube->C), alpha(1.0f), beta(0.0f), p_driver(_p_driver) {}

  void compute(const CubeType *const p_input1_cube, const CubeType *const p_input2_cube,
               CubeType *const p_output_cube) {
    int M = 0, N = 0, K = 0, LDA = 0, LDB = 0;
    CBLAS_TRANSPOSE TA = CblasNoTrans, TB = CblasNoTrans;
    switch (KERNELCONFIG) {
      case KernelConfig_GEMM_NOTRANS_NOTRANS:
        M = i1R; N = i2C; K = i1C; LDA = i1C; LDB = i2C; break;
      case KernelConfig_GEMM_NOTRANS_TRANS:
        TB = CblasTrans; M = i1R; N = i2R; K = i1C; LDA = i1C; LDB = i2C; break;
      case KernelConfig_GEMM_TRANS_NOTRANS:
        TA = CblasTrans; M = i1C; N = i2C; K = i1R; LDA = i1C; LDB = i2C; break;
      case KernelConfig_GEMM_NOTRANS_TRANS_NO_DIM_FLIP:
        TB = CblasTrans; M = i1R; N = i2C; K = i1C; LDA = i1C; LDB = i1C; break;
      case KernelConfig_GEMM_TRANS_NO_DIM_FLIP_NOTRANS:
        TA = CblasTrans; M = i1R; N = i2C; K = i1C; LDA = i2C; LDB = i2C; break;
      case KernelConfig_GEMM_NOTRANS_NOTRANS_DIM_FLIP:
        M = i1R; N = i2R; K = i1C; LDA = i1C; LDB = i2R; break;
      case KernelConfig_GEMM_NOTRANS_DIM_FLIP_NOTRANS:
        M = i1C; N = i2C; K = i1R; LDA = i1R; LDB = i2C; break;
    }
    p_driver->sgemm(CblasRowMajor, TA, TB, M, N, K, alpha, p_input1_cube->get_p_data(), LDA,
                    p_input2_cube->get_p_data(), LDB, beta, p_output_cube->get_p_data(), N);
  }

 private:
  DriverClass *p_driver;
};

}  // namespace cct
