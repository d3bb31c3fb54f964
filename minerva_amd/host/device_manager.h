// Owner of the devices of a process (reference minerva/device/device_manager.h:9-26,
// device_manager.cpp:14-75): creates GPU devices by index, hands them out by id, forwards a
// datum's release to every device that may hold it.  The reference's CreateGpuDevice makes a
// CUDA GpuDevice; here it makes a HipDevice.  There is no CPU device in this layer (the CPU
// implementation stays the reference's own), so CreateCpuDevice fails with an error.
#pragma once
#include <cstddef>
#include <cstdint>
#include <unordered_map>

#include "device.h"

namespace minerva {

class DeviceManager {
 public:
  // gpu_pool_bytes: what every GPU device's data store may keep cached (0: the device's default)
  explicit DeviceManager(size_t gpu_pool_bytes = 0);
  ~DeviceManager();
  uint64_t CreateCpuDevice();
  uint64_t CreateGpuDevice(int gid);
  int GetGpuDeviceCount();
  Device* GetDevice(uint64_t id);
  void FreeData(uint64_t id);
  void RegisterListener(DeviceListener* l) { listener_ = l; }

 private:
  uint64_t GenerateDeviceId();
  DeviceListener* listener_ = nullptr;
  std::unordered_map<uint64_t, Device*> device_storage_;
  size_t gpu_pool_bytes_;
  uint64_t next_device_id_ = 0;  // per manager; the reference counts in a function-local static
  DeviceManager(const DeviceManager&) = delete;
  DeviceManager& operator=(const DeviceManager&) = delete;
};

}  // namespace minerva
