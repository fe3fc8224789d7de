// Type-1 lowering connector: fills the argument structs and calls the driver.
// Counterpart of Connector<..., LOWERING_TYPE1, DriverClass>
// (src/Connector_impl_Lowering_type1.hxx:46-183).
#pragma once
#include <algorithm>
#include <cassert>

#include "LogicalCube.h"

namespace cct {

template <typename DataType, typename DriverClass>
class Connector {
 public:
  typedef LogicalCube<DataType> InputLogicalCubeType;
  typedef LogicalCube<DataType> OutputLogicalCubeType;

  const size_t iR, iC, iD, iB;
  const size_t oR, oC, oD, oB;
  const size_t kernel_size, padding, stride;

  Connector(const InputLogicalCubeType *const p_input_cube, const OutputLogicalCubeType *const p_output_cube,
            const size_t _kernel_size, const size_t _padding, const size_t _stride, DriverClass *_p_driver)
      : iR(p_input_cube->R), iC(p_input_cube->C), iD(p_input_cube->D), iB(p_input_cube->B),
        oR(p_output_cube->R), oC(p_output_cube->C), oD(p_output_cube->D), oB(p_output_cube->B),
        kernel_size(_kernel_size), padding(_padding), stride(_stride), p_driver(_p_driver) {
    // lowered cube is (k*k*d) x (m*m*b), Connector_impl_Lowering_type1.hxx:37-40
    assert(oD == 1 && oB == 1);
    assert(oR == kernel_size * kernel_size * iD);
    assert(oC == ((iR + 2 * padding - kernel_size) / stride + 1) * ((iC + 2 * padding - kernel_size) / stride + 1) * iB);
  }

  void lower_cube(const InputLogicalCubeType *const p_input_cube, OutputLogicalCubeType *p_output_cube) {
    DeviceMemoryPointer input = p_input_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_cube->get_device_pointer(p_driver);
    PMapHelper args = {};
    args.dR = p_output_cube->R; args.dC = p_output_cube->C; args.dD = p_output_cube->D; args.dB = p_output_cube->B;
    args.sR = p_input_cube->R; args.sC = p_input_cube->C; args.sD = p_input_cube->D; args.sB = p_input_cube->B;
    args.dBR = args.dR; args.dBC = args.dC;
    args.sBR = std::min((size_t)16, args.sR); args.sBC = std::min((size_t)16, args.sC);
    args.kR = kernel_size; args.kC = kernel_size; args.kD = p_input_cube->D; args.kB = 1;
    args.stride = stride;
    args.padding = padding;
    p_driver->lower_cube(&output, &input, args);
  }

  // [depth][batch] slices of `src` -> [batch][depth] slices of `dst` (out of place; the reference
  // copies the cube and permutes back into it, Connector_impl_Lowering_type1.hxx:92-128)
  // With `bias_grad` (backward pass, `batch` = number of maps) the same pass also leaves the maps'
  // bias gradient there.
  void remap_output(LogicalCube<DataType> &dst, const LogicalCube<DataType> &src, const size_t depth,
                    const size_t batch, const LogicalCube<DataType> *bias_grad = nullptr) {
    DeviceMemoryPointer d = dst.get_device_pointer(p_driver);
    DeviceMemoryPointer s = src.get_device_pointer(p_driver);
    PMapHelper args = {};
    args.dR = src.R; args.dC = src.C; args.dD = src.D; args.dB = src.B;
    args.sR = src.R; args.sC = src.C; args.sD = depth; args.sB = batch;
    args.dBR = args.dR; args.dBC = args.dC;
    args.sBR = std::min((size_t)16, args.sR); args.sBC = std::min((size_t)16, args.sC);
    args.stride = stride;
    args.padding = padding;
    if (bias_grad) {
      DeviceMemoryPointer b = bias_grad->get_device_pointer(p_driver);
      p_driver->pmap2d_read_coalesce_remap_bias_backward(&d, &s, args, &b);
    } else {
      p_driver->pmap2d_read_coalesce_remap(&d, &s, args);
    }
  }

  _inverse_lower_cube_arg_helper inverse_args() const {
    _inverse_lower_cube_arg_helper _arg;
    _arg.data_output_width = (iR + 2 * padding - kernel_size) / stride + 1;
    _arg.data_output_height = (iC + 2 * padding - kernel_size) / stride + 1;
    _arg.kernel_size = kernel_size;
    _arg.stride = stride;
    _arg.padding = padding;
    _arg.iR = iR; _arg.iC = iC; _arg.iD = iD; _arg.iB = iB;
    return _arg;
  }

  // p_output_cube: lowered gradient [k*k*d][b*m*m]; p_input_cube: input gradient.  The gather
  // kernel overwrites its destination, so the zero fill of the reference (:156) is not issued.
  void inverse_lower_cube(OutputLogicalCubeType *p_output_cube, InputLogicalCubeType *p_input_cube) {
    DeviceMemoryPointer input = p_input_cube->get_device_pointer(p_driver);
    DeviceMemoryPointer output = p_output_cube->get_device_pointer(p_driver);
    p_driver->inverse_lower_cube(&input, &output, inverse_args());
  }

 private:
  DriverClass *p_driver;
};

}  // namespace cct
