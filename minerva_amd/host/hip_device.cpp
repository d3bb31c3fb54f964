#include "hip_device.h"

#include <cstdio>

#include "mnv_hip.h"

namespace minerva {

namespace {
void Ok(int status, const char* what) {
  MNV_CHECK(status == MNV_OK) << what << ": " << mnv_error_string(status);
}
// Scratch arena per worker stream: split-k partial sums of the skinny GEMMs and of the
// convolution filter gradient.  The kernels use as many k ranges as fit.
constexpr size_t kWorkspaceBytes = (size_t)128 << 20;
}  // namespace

// ---------------------------------------------------------------- PooledDataStore

PooledDataStore::PooledDataStore(size_t threshold, std::function<void*(size_t)> a,
                                 std::function<void(void*)> d)
    : allocator_(std::move(a)), deallocator_(std::move(d)), threshold_(threshold) {}

PooledDataStore::~PooledDataStore() {
  for (auto& kv : data_states_) deallocator_(kv.second.ptr);
  for (auto& kv : free_space_)
    while (!kv.second.empty()) {
      deallocator_(kv.second.front());
      kv.second.pop();
    }
}

float* PooledDataStore::CreateData(uint64_t id, size_t length) {
  std::lock_guard<std::mutex> lck(access_mutex_);
  auto it = data_states_.emplace(id, DataState{nullptr, length});
  MNV_CHECK(it.second) << "data already existed";
  DataState& ds = it.first->second;
  auto hit = free_space_.find(length);
  if (hit != free_space_.end()) {  // reuse a block of exactly this size
    ds.ptr = hit->second.front();
    hit->second.pop();
    if (hit->second.empty()) free_space_.erase(hit);
  } else {
    ds.ptr = allocator_(length);
    total_ += length;
    if (threshold_ < total_) ReleaseFreeSpace();
  }
  return static_cast<float*>(ds.ptr);
}

float* PooledDataStore::GetData(uint64_t id) {
  std::lock_guard<std::mutex> lck(access_mutex_);
  auto it = data_states_.find(id);
  MNV_CHECK(it != data_states_.end()) << "data #" << id << " does not exist";
  return static_cast<float*>(it->second.ptr);
}

bool PooledDataStore::ExistData(uint64_t id) const {
  std::lock_guard<std::mutex> lck(access_mutex_);
  return data_states_.count(id) != 0;
}

void PooledDataStore::FreeData(uint64_t id) {
  std::lock_guard<std::mutex> lck(access_mutex_);
  auto it = data_states_.find(id);
  MNV_CHECK(it != data_states_.end()) << "data #" << id << " does not exist";
  free_space_[it->second.length].push(it->second.ptr);
  data_states_.erase(it);
}

size_t PooledDataStore::GetTotalBytes() const {
  std::lock_guard<std::mutex> lck(access_mutex_);
  return total_;
}

size_t PooledDataStore::NumCachedBlocks() const {
  std::lock_guard<std::mutex> lck(access_mutex_);
  size_t n = 0;
  for (auto& kv : free_space_) n += kv.second.size();
  return n;
}

void PooledDataStore::ReleaseFreeSpace() {
  for (auto& kv : free_space_)
    while (!kv.second.empty()) {
      deallocator_(kv.second.front());
      kv.second.pop();
      total_ -= kv.first;
    }
  free_space_.clear();
}

// ---------------------------------------------------------------------- HipDevice

HipDevice::HipDevice(uint64_t device_id, DeviceListener* listener, int gpu_id, size_t pool_bytes)
    : device_id_(device_id), listener_(listener), gpu_id_(gpu_id) {
  Activate();
  for (size_t i = 0; i < kParallelism; ++i) Ok(mnv_stream_create(&streams_[i]), "stream create");
  auto allocator = [this](size_t len) -> void* {
    void* p = nullptr;
    MNV_CHECK(!capturing_) << "a block of " << len << " bytes is not cached: device memory "
                           << "cannot be allocated while a graph is recorded";
    Activate();
    Ok(mnv_malloc(&p, len), "device malloc");
    return p;
  };
  auto deallocator = [this](void* p) {
    Activate();
    // A cached block may still be read by a kernel in flight when operators are not
    // synchronised one by one; hipFree itself waits for the device, so this is safe.
    mnv_free(p);
  };
  data_store_.reset(new PooledDataStore(pool_bytes, allocator, deallocator));
  for (size_t i = 0; i < kParallelism; ++i)
    workers_.emplace_back(&HipDevice::WorkerLoop, this, static_cast<int>(i));
}

HipDevice::~HipDevice() {
  WaitForAllFinished();
  {
    std::lock_guard<std::mutex> lck(q_mutex_);
    stop_ = true;
  }
  q_cv_.notify_all();
  for (auto& t : workers_) t.join();
  Activate();
  for (size_t i = 0; i < kParallelism; ++i) mnv_stream_sync(streams_[i]);
  data_store_.reset();  // before the streams: the deallocator uses the device
  for (size_t i = 0; i < kParallelism; ++i) {
    if (workspace_[i]) mnv_free(workspace_[i]);
    mnv_stream_destroy(streams_[i]);
  }
}

void HipDevice::Activate() const { Ok(mnv_device_set(gpu_id_), "set device"); }

std::string HipDevice::Name() const {
  char buf[64];
  snprintf(buf, sizeof(buf), "HIP device #%d", static_cast<int>(device_id_));
  return buf;
}

std::string HipDevice::GetMemUsage() const {
  char buf[96];
  snprintf(buf, sizeof(buf), "device #%d used %zuB", static_cast<int>(device_id_),
           data_store_->GetTotalBytes());
  return buf;
}

std::pair<HipDevice::MemType, float*> HipDevice::GetPtr(uint64_t data_id) {
  return std::make_pair(MemType::kGpu, data_store_->GetData(data_id));
}

void HipDevice::FreeDataIfExist(uint64_t data_id) {
  size_t erased;
  {
    std::lock_guard<std::mutex> lck(local_mutex_);
    erased = local_data_.erase(data_id);
  }
  if (erased == 1) data_store_->FreeData(data_id);
}

void HipDevice::PushTask(Task* task) {
  if (task->light) {
    Execute(task, 0);  // light tasks skip the thread hop (device.cpp:55-61)
    return;
  }
  {
    std::lock_guard<std::mutex> lck(q_mutex_);
    queue_.push_back(task);
  }
  q_cv_.notify_one();
}

void HipDevice::WorkerLoop(int thrid) {
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
      std::lock_guard<std::mutex> lck(err_mutex_);
      if (async_error_.empty()) async_error_ = e.what();
      if (listener_) listener_->OnOperationComplete(task);
    }
    {
      std::lock_guard<std::mutex> lck(q_mutex_);
      --busy_;
    }
    idle_cv_.notify_all();
  }
}

void HipDevice::WaitForAllFinished() {
  std::unique_lock<std::mutex> lck(q_mutex_);
  idle_cv_.wait(lck, [this] { return queue_.empty() && busy_ == 0; });
}

std::string HipDevice::TakeAsyncError() {
  std::lock_guard<std::mutex> lck(err_mutex_);
  std::string e;
  e.swap(async_error_);
  return e;
}

void HipDevice::EnsureWorkspace(int thrid, size_t bytes) {
  if (workspace_bytes_[thrid] >= bytes) return;
  if (workspace_[thrid]) {
    Ok(mnv_stream_sync(streams_[thrid]), "workspace sync");
    Ok(mnv_free(workspace_[thrid]), "workspace free");
  }
  Ok(mnv_malloc(&workspace_[thrid], bytes), "workspace malloc");
  workspace_bytes_[thrid] = bytes;
}

void HipDevice::Execute(Task* task, int thrid) {
  Activate();  // every task re-selects the device on its thread (device.cpp:201-203)
  DataList input_shards;
  for (auto& i : task->inputs) {
    auto& d = i.physical_data;
    // One GPU: every input is local.  A remote input would be copied here with
    // mnv_memcpy_d2d over xGMI, as DoCopyRemoteData does in the reference.
    MNV_CHECK_EQ(d.device_id, device_id_) << "remote inputs are not part of the one-GPU build";
    {
      std::lock_guard<std::mutex> lck(local_mutex_);
      MNV_CHECK_EQ(local_data_.count(d.data_id), 1u) << "input data #" << d.data_id << " missing";
    }
    input_shards.emplace_back(data_store_->GetData(d.data_id), d.size);
  }
  DataList output_shards;
  for (auto& o : task->outputs) {
    size_t bytes = static_cast<size_t>(o.physical_data.size.Prod()) * sizeof(float);
    float* ptr = data_store_->CreateData(o.physical_data.data_id, bytes);
    {
      std::lock_guard<std::mutex> lck(local_mutex_);
      MNV_CHECK(local_data_.insert(o.physical_data.data_id).second) << "duplicate data";
    }
    output_shards.emplace_back(ptr, o.physical_data.size);
  }
  MNV_CHECK(task->op.compute_fn) << "task without an operator";
  DoExecute(input_shards, output_shards, task->op, thrid);
  if (listener_) listener_->OnOperationComplete(task);
}

void HipDevice::DoExecute(const DataList& in, const DataList& out, PhysicalOp& op, int thrid) {
  EnsureWorkspace(thrid, kWorkspaceBytes);
  Context ctx;
  ctx.impl_type = ImplType::kHip;
  ctx.stream = streams_[thrid];
  ctx.workspace = workspace_[thrid];
  ctx.workspace_bytes = workspace_bytes_[thrid];
  Timed t{std::string(), nullptr, nullptr};
  const bool timed = profile_ && !capturing_;
  if (timed) {
    t.name = op.compute_fn->Name();
    Ok(mnv_event_create(&t.start), "event create");
    Ok(mnv_event_create(&t.stop), "event create");
    Ok(mnv_event_record(t.start, streams_[thrid]), "event record");
  }
  op.compute_fn->Execute(in, out, ctx);
  if (timed) {
    Ok(mnv_event_record(t.stop, streams_[thrid]), "event record");
    std::lock_guard<std::mutex> lck(prof_mutex_);
    timed_.push_back(t);
  }
  if (sync_each_op_ && !capturing_) {
    int rc = mnv_stream_sync(streams_[thrid]);
    MNV_CHECK(rc == MNV_OK) << op.compute_fn->Name() << ": " << mnv_error_string(rc);
  }
}

std::map<std::string, std::pair<int, double>> HipDevice::CollectProfile() {
  Activate();
  for (size_t i = 0; i < kParallelism; ++i) Ok(mnv_stream_sync(streams_[i]), "profile sync");
  std::vector<Timed> rec;
  {
    std::lock_guard<std::mutex> lck(prof_mutex_);
    rec.swap(timed_);
  }
  std::map<std::string, std::pair<int, double>> out;
  for (auto& t : rec) {
    float ms = 0.f;
    Ok(mnv_event_elapsed_ms(t.start, t.stop, &ms), "event elapsed");
    auto& e = out[t.name];
    e.first += 1;
    e.second += ms;
    mnv_event_destroy(t.start);
    mnv_event_destroy(t.stop);
  }
  return out;
}

void HipDevice::BeginCapture() {
  MNV_CHECK(!capturing_) << "a graph is already being recorded";
  WaitForAllFinished();
  Activate();
  EnsureWorkspace(0, kWorkspaceBytes);
  for (size_t i = 0; i < kParallelism; ++i) Ok(mnv_stream_sync(streams_[i]), "capture sync");
  Ok(mnv_graph_begin_capture(streams_[0]), "begin capture");
  capturing_ = true;
}

void* HipDevice::EndCapture(size_t* num_nodes) {
  MNV_CHECK(capturing_) << "no graph is being recorded";
  capturing_ = false;
  void* exec = nullptr;
  int rc = mnv_graph_end_capture(streams_[0], &exec, num_nodes);
  if (rc != MNV_OK) mnv_graph_abort_capture(streams_[0]);
  Ok(rc, "end capture");
  return exec;
}

void HipDevice::AbortCapture() {
  if (!capturing_) return;
  capturing_ = false;
  mnv_graph_abort_capture(streams_[0]);
}

void HipDevice::LaunchGraph(void* graph_exec) {
  MNV_CHECK(!capturing_) << "a graph cannot be replayed while another is recorded";
  Activate();
  Ok(mnv_graph_launch(graph_exec, streams_[0]), "graph launch");
}

void HipDevice::Barrier(int thrid) {
  MNV_CHECK(!capturing_) << "no synchronisation while a graph is recorded";
  Ok(mnv_stream_sync(streams_[thrid]), "barrier");
}

void HipDevice::CopyToHost(float* dst, uint64_t data_id, size_t floats) {
  MNV_CHECK(!capturing_) << "no host copies while a graph is recorded";
  Activate();
  Ok(mnv_memcpy_d2h(dst, data_store_->GetData(data_id), floats * sizeof(float), streams_[0]),
     "copy to host");
  Ok(mnv_stream_sync(streams_[0]), "copy to host sync");
}

void HipDevice::CopyFromHost(uint64_t data_id, const float* src, size_t floats) {
  MNV_CHECK(!capturing_) << "no host copies while a graph is recorded";
  Activate();
  Ok(mnv_memcpy_h2d(data_store_->GetData(data_id), src, floats * sizeof(float), streams_[0]),
     "copy from host");
  Ok(mnv_stream_sync(streams_[0]), "copy from host sync");
}

void HipDevice::CopyOnDevice(uint64_t dst_id, uint64_t src_id, size_t floats) {
  Activate();
  Ok(mnv_copy(data_store_->GetData(src_id), data_store_->GetData(dst_id), floats, streams_[0]),
     "device copy");
}

}  // namespace minerva
