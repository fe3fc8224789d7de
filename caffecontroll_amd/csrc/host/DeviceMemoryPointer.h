// Tagged pointer handed between bridges and drivers.
// Counterpart of src/sched/DeviceMemoryPointer.h:13-18,53-88: {ptr, size_in_byte, type}.  The
// reference's cross-device deref/write_through hooks are not needed on this path (one device,
// tensors stay resident) and are left out.
#pragma once
#include <cstddef>

namespace cct {

enum DeviceMemoryType {
  DEVICEMEMORY_LOCAL_RAM = 0,
  DEVICEMEMORY_QPI_RAM = 1,
  DEVICEMEMORY_LOCAL_GPURAM = 2,
  DEVICEMEMORY_REMOTE_RAM = 3
};

struct DeviceMemoryPointer {
  void *ptr;
  size_t size_in_byte;
  DeviceMemoryType type;
  DeviceMemoryPointer(void *_ptr, size_t _size_in_byte, DeviceMemoryType _type)
      : ptr(_ptr), size_in_byte(_size_in_byte), type(_type) {}
};

struct DeviceMemoryPointer_Local_RAM : DeviceMemoryPointer {
  DeviceMemoryPointer_Local_RAM(void *_ptr, size_t _size_in_byte)
      : DeviceMemoryPointer(_ptr, _size_in_byte, DEVICEMEMORY_LOCAL_RAM) {}
};

struct DeviceMemoryPointer_Local_GPURAM : DeviceMemoryPointer {
  DeviceMemoryPointer_Local_GPURAM(void *_ptr, size_t _size_in_byte)
      : DeviceMemoryPointer(_ptr, _size_in_byte, DEVICEMEMORY_LOCAL_GPURAM) {}
};

}  // namespace cct
