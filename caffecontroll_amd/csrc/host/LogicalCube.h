// 4-D tensor view in the reference's Layout_CRDB (src/LogicalCube.h:44-221): physical index
// c + r*C + d*R*C + b*R*C*D, i.e. dense NCHW.  Cubes on this path live in device memory.
#pragma once
#include <cassert>
#include <cstddef>

#include "DeviceMemoryPointer.h"
#include "HIPDriver.h"

namespace cct {

template <typename T>
class LogicalCube {
 public:
  const size_t n_elements;
  const size_t R, C, D;
  size_t B;
  bool own_data;

  // points to existing (device) data, does not own it -- LogicalCube.h:58-62
  LogicalCube(void *_p_data, size_t _R, size_t _C, size_t _D, size_t _B)
      : n_elements(_R * _C * _D * _B), R(_R), C(_C), D(_D), B(_B), own_data(false),
        p_data(reinterpret_cast<T *>(_p_data)), p_driver(nullptr) {}

  // allocates on the device through the driver and owns the memory -- LogicalCube.h:95-96
  LogicalCube(size_t _R, size_t _C, size_t _D, size_t _B, HIPDriver *_p_driver)
      : n_elements(_R * _C * _D * _B), R(_R), C(_C), D(_D), B(_B), own_data(true), p_data(nullptr),
        p_driver(_p_driver) {
    DeviceMemoryPointer_Local_GPURAM mem(nullptr, n_elements * sizeof(T));
    p_driver->malloc(&mem);
    p_data = reinterpret_cast<T *>(mem.ptr);
  }

  ~LogicalCube() {
    if (own_data && p_data) {
      DeviceMemoryPointer_Local_GPURAM mem(p_data, n_elements * sizeof(T));
      p_driver->free(&mem);
    }
  }
  LogicalCube(const LogicalCube &) = delete;
  LogicalCube &operator=(const LogicalCube &) = delete;

  T *get_p_data() const { return p_data; }

  // only for non-owning cubes (src/LogicalCube_impl.hxx:20-33 frees owned memory instead; here
  // re-pointing an owning cube is refused)
  void set_p_data(T *const data) {
    assert(!own_data);
    p_data = data;
  }

  // Becomes a non-owning view of `data` (same shape), releasing the memory the cube owned, if any: how a
  // bridge's own device cube turns into an alias of its neighbour's once the two are told to share.
  void adopt(T *const data) {
    if (own_data && p_data) {
      DeviceMemoryPointer_Local_GPURAM mem(p_data, n_elements * sizeof(T));
      p_driver->free(&mem);
    }
    own_data = false;
    p_data = data;
  }

  // The reference returns a heap wrapper that is never freed (src/LogicalCube.h:64-66); this
  // returns the wrapper by value.
  DeviceMemoryPointer get_device_pointer(HIPDriver *driver) const {
    return driver->get_device_pointer(p_data, n_elements * sizeof(T));
  }
  DeviceMemoryPointer get_device_pointer_RCDslice(HIPDriver *driver, size_t b_offset, size_t num_batches) const {
    assert(b_offset + num_batches <= B);
    return driver->get_device_pointer(p_data + b_offset * R * C * D, num_batches * R * C * D * sizeof(T));
  }

 private:
  T *p_data;
  HIPDriver *p_driver;
};

// A layer is a data cube plus its gradient cube (src/Layer.h:24-62).
template <typename T>
class Layer {
 public:
  typedef LogicalCube<T> DataLogicalCubeType;
  typedef LogicalCube<T> GradientLogicalCubeType;
  DataLogicalCubeType *const p_data_cube;
  GradientLogicalCubeType *const p_gradient_cube;
  const size_t dR, dC, dD, dB;
  const size_t gR, gC, gD, gB;

  Layer(DataLogicalCubeType *_p_data_cube, GradientLogicalCubeType *_p_gradient_cube)
      : p_data_cube(_p_data_cube), p_gradient_cube(_p_gradient_cube), dR(_p_data_cube->R),
        dC(_p_data_cube->C), dD(_p_data_cube->D), dB(_p_data_cube->B), gR(_p_gradient_cube->R),
        gC(_p_gradient_cube->C), gD(_p_gradient_cube->D), gB(_p_gradient_cube->B) {
    assert(dR == gR && dC == gC && dD == gD && dB == gB);
  }
  ~Layer() {
    delete p_data_cube;
    delete p_gradient_cube;
  }
};

}  // namespace cct
