// The device interface the engine drives, with the reference's class layering and member
// functions (minerva/device/device.h:18-63, device/task.h:9-19, device/task_data.h,
// device/device_listener.h:6-10, op/physical.h, op/compute_fn.h:9-12):
//   Device           PushTask / GetPtr / FreeDataIfExist / GetMemUsage / Name / GetMemType
//   ThreadedDevice   a pool of `parallelism` worker threads; Execute(Task*, thrid) prepares the
//                    operands in the data store and calls the hooks a concrete device overrides:
//                    PreExecute, Barrier, DoCopyRemoteData, DoExecute
// HipDevice (hip_device.h) is the GPU subclass, where the reference has GpuDevice.  Nothing
// in this file touches a GPU: the CPU tests of the host layer derive a malloc-backed device
// from ThreadedDevice and run it under the address and thread sanitizers.
#pragma once
#include <condition_variable>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_set>
#include <utility>
#include <vector>

#include "minerva_types.h"
#include "pooled_data_store.h"

namespace minerva {

// What a task runs: an operator with its closure bound (reference op/compute_fn.h:9-12).
class ComputeFn {
 public:
  virtual ~ComputeFn() {}
  virtual void Execute(const DataList&, const DataList&, const Context&) = 0;
  virtual std::string Name() const = 0;
  // Index of an input the operator writes (LRNForward fills its `scale` input, as the
  // reference does, cuda.cpp:45-59), or -1: a device that orders operators by data
  // dependencies must treat the operator as that datum's latest producer.
  virtual int MutatedInput() const { return -1; }
};

struct PhysicalData {
  PhysicalData(const Scale& s, uint64_t d, uint64_t id) : size(s), device_id(d), data_id(id) {}
  Scale size;
  uint64_t device_id;
  uint64_t data_id;
};

struct PhysicalOp {
  std::shared_ptr<ComputeFn> compute_fn;
  uint64_t device_id = 0;
};

struct TaskData {
  TaskData(const PhysicalData& p, uint64_t i) : physical_data(p), id(i) {}
  PhysicalData physical_data;
  uint64_t id;
};

struct Task {
  std::vector<TaskData> inputs;
  std::vector<TaskData> outputs;
  PhysicalOp op;
  uint64_t id = 0;     // only meaningful to the issuer of the task
  bool light = false;  // run on the caller's thread instead of the pool
  int stream = 0;      // light tasks: which worker stream (0 unless the device is in dataflow mode)
};

class DeviceListener {
 public:
  virtual ~DeviceListener() = default;
  virtual void OnOperationComplete(Task*) = 0;
};

class Device {
 public:
  enum class MemType { kCpu, kGpu };
  Device() = delete;
  Device(const Device&) = delete;
  Device& operator=(const Device&) = delete;
  Device(uint64_t device_id, DeviceListener*);
  virtual ~Device() = default;
  virtual void PushTask(Task*) = 0;
  virtual std::pair<MemType, float*> GetPtr(uint64_t data_id);
  virtual void FreeDataIfExist(uint64_t data_id);
  virtual std::string GetMemUsage() const;
  virtual std::string Name() const = 0;
  virtual MemType GetMemType() const = 0;
  uint64_t device_id() const { return device_id_; }

 protected:
  // ids of the data this device holds (the reference's ConcurrentUnorderedSet)
  class IdSet {
   public:
    bool Insert(uint64_t id) {
      std::lock_guard<std::mutex> lck(m_);
      return s_.insert(id).second;
    }
    size_t Erase(uint64_t id) {
      std::lock_guard<std::mutex> lck(m_);
      return s_.erase(id);
    }
    size_t Count(uint64_t id) const {
      std::lock_guard<std::mutex> lck(m_);
      return s_.count(id);
    }

   private:
    mutable std::mutex m_;
    std::unordered_set<uint64_t> s_;
  };
  IdSet local_data_;
  IdSet remote_data_;
  uint64_t device_id_;
  std::unique_ptr<PooledDataStore> data_store_;
  DeviceListener* listener_;
};

class ThreadedDevice : public Device {
 public:
  ThreadedDevice() = delete;
  ThreadedDevice(uint64_t device_id, DeviceListener*, size_t parallelism);
  ~ThreadedDevice() override;
  void PushTask(Task*) override;
  void FreeDataIfExist(uint64_t data_id) override;
  // Blocks until the pool has run every task pushed so far.
  void WaitForAllFinished();
  // First error raised by an operator on a pool thread (empty if none): the reference
  // aborts the process there; here the listener is still told and the error is kept.
  std::string TakeAsyncError();

 protected:
  virtual void Execute(Task*, int thrid);
  virtual void PreExecute();
  virtual void Barrier(int);
  virtual void DoCopyRemoteData(float*, float*, size_t, int) = 0;
  virtual void DoExecute(const DataList&, const DataList&, PhysicalOp&, int) = 0;
  // True on a thread of this device's pool (a task pushed with light == false).
  static bool OnPoolThread();
  // Ends the pool: called by the destructor, and earlier by a subclass whose hooks use
  // resources that its own destructor releases.
  void StopWorkers();

 private:
  void WorkerLoop(int thrid);
  std::vector<std::thread> workers_;
  std::mutex q_mutex_;
  std::condition_variable q_cv_, idle_cv_;
  std::deque<Task*> queue_;
  size_t busy_ = 0;
  bool stop_ = false;
  std::mutex err_mutex_;
  std::string async_error_;
};

}  // namespace minerva
