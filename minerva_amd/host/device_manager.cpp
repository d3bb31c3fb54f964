#include "device_manager.h"

#include "hip_device.h"
#include "mnv_hip.h"

namespace minerva {

DeviceManager::DeviceManager(size_t gpu_pool_bytes) : gpu_pool_bytes_(gpu_pool_bytes) {}

DeviceManager::~DeviceManager() {
  for (auto& i : device_storage_) delete i.second;
}

uint64_t DeviceManager::CreateCpuDevice() {
  MNV_CHECK(false) << "no CPU device in the HIP host layer: the CPU implementation is the reference's";
  return 0;
}

uint64_t DeviceManager::CreateGpuDevice(int gid) {
  MNV_CHECK(gid >= 0 && gid < GetGpuDeviceCount()) << "no GPU #" << gid;
  const uint64_t id = GenerateDeviceId();
  Device* d = gpu_pool_bytes_ ? new HipDevice(id, listener_, gid, gpu_pool_bytes_)
                              : new HipDevice(id, listener_, gid);
  MNV_CHECK(device_storage_.emplace(id, d).second) << "duplicate device id";
  return id;
}

int DeviceManager::GetGpuDeviceCount() {
  int count = 0;
  const int rc = mnv_device_count(&count);
  MNV_CHECK(rc == MNV_OK) << "device count: " << mnv_error_string(rc);
  return count;
}

Device* DeviceManager::GetDevice(uint64_t id) {
  auto it = device_storage_.find(id);
  MNV_CHECK(it != device_storage_.end()) << "no device #" << id;
  return it->second;
}

void DeviceManager::FreeData(uint64_t id) {
  for (auto& i : device_storage_) i.second->FreeDataIfExist(id);
}

uint64_t DeviceManager::GenerateDeviceId() { return next_device_id_++; }

}  // namespace minerva
