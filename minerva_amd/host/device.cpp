#include "device.h"

#include <cstdio>

namespace minerva {

Device::Device(uint64_t device_id, DeviceListener* l) : device_id_(device_id), listener_(l) {}

std::pair<Device::MemType, float*> Device::GetPtr(uint64_t data_id) {
  return std::make_pair(GetMemType(), data_store_->GetData(data_id));
}

void Device::FreeDataIfExist(uint64_t data_id) {
  size_t d = local_data_.Erase(data_id) + remote_data_.Erase(data_id);
  if (d == 1) data_store_->FreeData(data_id);
  else MNV_CHECK(d == 0) << "duplicate data";
}

std::string Device::GetMemUsage() const {
  char buf[96];
  snprintf(buf, sizeof(buf), "device #%d used %zuB", static_cast<int>(device_id_),
           data_store_->GetTotalBytes());
  return buf;
}

// ------------------------------------------------------------------ ThreadedDevice

namespace {
thread_local bool tl_on_pool_thread = false;
}

ThreadedDevice::ThreadedDevice(uint64_t device_id, DeviceListener* l, size_t parallelism)
    : Device(device_id, l) {
  for (size_t i = 0; i < parallelism; ++i)
    workers_.emplace_back(&ThreadedDevice::WorkerLoop, this, static_cast<int>(i));
}

ThreadedDevice::~ThreadedDevice() { StopWorkers(); }

void ThreadedDevice::StopWorkers() {
  if (workers_.empty()) return;
  WaitForAllFinished();
  {
    std::lock_guard<std::mutex> lck(q_mutex_);
    stop_ = true;
  }
  q_cv_.notify_all();
  for (auto& t : workers_) t.join();
  workers_.clear();
}

bool ThreadedDevice::OnPoolThread() { return tl_on_pool_thread; }

void ThreadedDevice::PushTask(Task* task) {
  if (task->light) {  // light tasks skip the thread hop (reference device.cpp:55-61)
    Execute(task, 0);
    return;
  }
  {
    std::lock_guard<std::mutex> lck(q_mutex_);
    queue_.push_back(task);
  }
  q_cv_.notify_one();
}

void ThreadedDevice::FreeDataIfExist(uint64_t data_id) { Device::FreeDataIfExist(data_id); }

void ThreadedDevice::WorkerLoop(int thrid) {
  tl_on_pool_thread = true;
  for (;;) {
    Task* task = nullptr;
    {
      std::unique_lock<std::mutex> lck(q_mutex_);
      q_cv_.wait(lck, [this] { return stop_ || !queue_.empty(); });
      if (queue_.empty()) return;  // stop_ and drained
      task = queue_.front();
      queue_.pop_front();
      ++busy_;
    }
    try {
      Execute(task, thrid);
    } catch (const std::exception& e) {
      {
        std::lock_guard<std::mutex> lck(err_mutex_);
        if (async_error_.empty()) async_error_ = e.what();
      }
      if (listener_) listener_->OnOperationComplete(task);
    }
    {
      std::lock_guard<std::mutex> lck(q_mutex_);
      --busy_;
    }
    idle_cv_.notify_all();
  }
}

void ThreadedDevice::WaitForAllFinished() {
  std::unique_lock<std::mutex> lck(q_mutex_);
  idle_cv_.wait(lck, [this] { return queue_.empty() && busy_ == 0; });
}

std::string ThreadedDevice::TakeAsyncError() {
  std::lock_guard<std::mutex> lck(err_mutex_);
  std::string e;
  e.swap(async_error_);
  return e;
}

// The reference's sequence (device.cpp:68-119): select the device, find or fetch every
// input, create every output in the data store, run the operator, tell the listener.
void ThreadedDevice::Execute(Task* task, int thrid) {
  PreExecute();
  DataList input_shards;
  for (auto& i : task->inputs) {
    auto& d = i.physical_data;
    // Every input is local in a one-device build.  A remote input would be created here
    // and filled by DoCopyRemoteData from the owning device's pointer.
    MNV_CHECK_EQ(d.device_id, device_id_) << "remote inputs are not part of the one-GPU build";
    MNV_CHECK_EQ(local_data_.Count(d.data_id), 1u) << "input data #" << d.data_id << " missing";
    input_shards.emplace_back(data_store_->GetData(d.data_id), d.size);
  }
  DataList output_shards;
  for (auto& o : task->outputs) {
    size_t bytes = static_cast<size_t>(o.physical_data.size.Prod()) * sizeof(float);
    float* ptr = data_store_->CreateData(o.physical_data.data_id, bytes);
    MNV_CHECK(local_data_.Insert(o.physical_data.data_id)) << "duplicate data";
    output_shards.emplace_back(ptr, o.physical_data.size);
  }
  MNV_CHECK(task->op.compute_fn) << "task without an operator";
  DoExecute(input_shards, output_shards, task->op, thrid);
  if (listener_) listener_->OnOperationComplete(task);
}

void ThreadedDevice::PreExecute() {}

void ThreadedDevice::Barrier(int) {}

}  // namespace minerva
