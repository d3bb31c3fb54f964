// The HIP device: the replacement for the reference's GpuDevice
// (minerva/device/device.h:18-78, device.cpp:129-222) and its allocator
// (minerva/device/pooled_data_store.cpp:19-65), with the same public surface the
// engine calls: PushTask / GetPtr / FreeDataIfExist and DeviceListener::OnOperationComplete.
//
//  - kParallelism (4) worker threads, each with its own HIP stream and its own
//    grow-only scratch arena; a task of the pool runs on worker `thrid` and, unless the
//    device is in dataflow mode, is synchronised before completion is reported, as the
//    reference does after every operator.
//  - PooledDataStore: exact-size free lists over mnv_malloc / mnv_free; when the bytes
//    held exceed the threshold every cached block is released.
//  - Three ways to order operators: synchronise after every one (the reference);
//    leave them in flight on one stream (stream order); or "dataflow": operators run on
//    any of the four streams, every output carries an event recorded behind its producer,
//    and a consumer on another stream waits for that event on the GPU, never on the host.
#pragma once
#include <array>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <queue>
#include <thread>
#include <unordered_map>
#include <unordered_set>

#include "op_dispatch.h"

namespace minerva {

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
  uint64_t id = 0;
  bool light = false;  // run on the caller's thread instead of the pool
  int stream = 0;      // light tasks: which worker stream (0 unless the device is in dataflow mode)
};

class DeviceListener {
 public:
  virtual ~DeviceListener() = default;
  virtual void OnOperationComplete(Task*) = 0;
};

class PooledDataStore {
 public:
  PooledDataStore(size_t threshold, std::function<void*(size_t)> a, std::function<void(void*)> d);
  ~PooledDataStore();
  PooledDataStore(const PooledDataStore&) = delete;
  PooledDataStore& operator=(const PooledDataStore&) = delete;
  // `stream` >= 0 (dataflow mode): prefer a cached block that only this stream has touched.
  // *foreign receives the streams (bit per stream) other than `stream` whose queued work may
  // still use the block handed out; the caller makes `stream` wait for them.
  float* CreateData(uint64_t id, size_t length, int stream = -1, unsigned* foreign = nullptr);
  float* GetData(uint64_t id);
  bool ExistData(uint64_t id) const;
  // `users`: the streams that have work queued on the block (0 when everything is known
  // to have finished).
  void FreeData(uint64_t id, unsigned users = 0);
  // Every queued operator has finished: cached blocks have no users left.
  void ClearUsers();
  size_t GetTotalBytes() const;
  size_t NumCachedBlocks() const;

 private:
  void ReleaseFreeSpace();
  struct DataState {
    void* ptr;
    size_t length;
  };
  mutable std::mutex access_mutex_;
  std::unordered_map<uint64_t, DataState> data_states_;
  struct FreeBlock {
    void* ptr;
    unsigned users;
  };
  std::unordered_map<size_t, std::deque<FreeBlock>> free_space_;
  std::function<void*(size_t)> allocator_;
  std::function<void(void*)> deallocator_;
  size_t threshold_;
  size_t total_ = 0;
};

class HipDevice {
 public:
  enum class MemType { kCpu, kGpu };
  static constexpr size_t kParallelism = 4;
  // 288 GB of HBM: keep up to 200 GiB in the pool before dropping cached blocks.
  static constexpr size_t kDefaultPoolBytes = (size_t)200 << 30;

  HipDevice(uint64_t device_id, DeviceListener* listener, int gpu_id,
            size_t pool_bytes = kDefaultPoolBytes);
  ~HipDevice();
  HipDevice(const HipDevice&) = delete;
  HipDevice& operator=(const HipDevice&) = delete;

  void PushTask(Task* task);
  std::pair<MemType, float*> GetPtr(uint64_t data_id);
  void FreeDataIfExist(uint64_t data_id);
  std::string GetMemUsage() const;
  std::string Name() const;
  MemType GetMemType() const { return MemType::kGpu; }
  void WaitForAllFinished();

  // When false, operators are left in flight on their stream and the caller decides
  // when to synchronise (Barrier); the reference always synchronises per operator.
  void set_sync_each_op(bool v) { sync_each_op_ = v; }
  // Dataflow mode: light tasks may name any worker stream; dependencies across streams
  // are kept by events on the GPU.  Implies no synchronisation per operator.
  void set_dataflow(bool v);
  bool dataflow() const { return dataflow_; }
  // Since the device was created: waits of a consumer's stream for a producer on another
  // stream, and waits of a stream for other streams before it reuses a recycled block.
  uint64_t producer_waits() const { return producer_waits_; }
  uint64_t recycle_waits() const { return recycle_waits_; }
  // Waits for worker stream `thrid`; in dataflow mode for all of them.
  void Barrier(int thrid);
  void* stream(int thrid) const { return streams_[thrid]; }
  uint64_t device_id() const { return device_id_; }
  PooledDataStore& data_store() { return *data_store_; }
  // Host <-> device copies on worker stream 0, synchronised.
  void CopyToHost(float* dst, uint64_t data_id, size_t floats);
  // Overwrites existing data in place (its address does not change).
  void CopyFromHost(uint64_t data_id, const float* src, size_t floats);
  // dst <- src on worker stream 0, left in flight (a kernel, so it can be recorded).
  void CopyOnDevice(uint64_t dst_id, uint64_t src_id, size_t floats);
  // First error raised by an operator on a pool thread (empty if none).
  std::string TakeAsyncError();

  // Per-operator timing, the counterpart of the reference's ExecutionProfiler
  // (minerva/profiler/execution_profiler.cpp:17-53): while enabled, every operator is
  // bracketed by two events on its own stream; CollectProfile synchronises and returns
  // name -> (launch count, total device milliseconds), then clears the record.
  void set_profile(bool v) { profile_ = v; }
  // Only operators whose name contains `part` are timed (empty: all).  Two events per
  // operator cost a few microseconds of GPU idle time each, so a measurement that wants
  // one kernel's duration inside an otherwise undisturbed step names that kernel.
  void set_profile_filter(const std::string& part) { profile_filter_ = part; }
  std::map<std::string, std::pair<int, double>> CollectProfile();

  // Records the light tasks pushed between Begin and End (they run on worker stream 0)
  // into a HIP graph instead of executing them.  While recording, operators are neither
  // synchronised nor timed, and the data store may only hand out cached blocks: a device
  // allocation cannot be recorded, so the caller runs the same task sequence once before
  // and keeps its blocks cached.  EndCapture returns the instantiated graph;
  // AbortCapture discards a recording that failed.  LaunchGraph replays on stream 0.
  void BeginCapture();
  void* EndCapture(size_t* num_nodes);
  void AbortCapture();
  bool capturing() const { return capturing_; }
  void LaunchGraph(void* graph_exec);

 private:
  // pooled: the task came through the thread pool (not issued inline by the caller)
  void Execute(Task* task, int thrid, bool pooled = false);
  void DoExecute(const DataList& in, const DataList& out, PhysicalOp& op, int thrid, bool pooled);
  void Activate() const;
  void EnsureWorkspace(int thrid, size_t bytes);
  void EnsureStaging(int thrid);
  void WorkerLoop(int thrid);

  uint64_t device_id_;
  DeviceListener* listener_;
  int gpu_id_;
  bool sync_each_op_ = true;
  bool capturing_ = false;
  bool dataflow_ = false;
  // dataflow mode, guarded by local_mutex_: where each datum was produced (stream, event
  // recorded behind the producer) and which streams have work queued that touches it
  struct Produced {
    void* event;
    int stream;
    unsigned users;
  };
  std::unordered_map<uint64_t, Produced> produced_;
  void WaitForStreams(int thrid, unsigned streams);
  std::atomic<uint64_t> producer_waits_{0}, recycle_waits_{0};
  std::array<void*, kParallelism> streams_{};
  std::array<void*, kParallelism> workspace_{};
  std::array<size_t, kParallelism> workspace_bytes_{};
  std::array<void*, kParallelism> staging_{};  // pinned host memory, allocated at first use
  std::unique_ptr<PooledDataStore> data_store_;
  std::mutex local_mutex_;
  std::unordered_set<uint64_t> local_data_;
  // thread pool
  std::vector<std::thread> workers_;
  std::mutex q_mutex_;
  std::condition_variable q_cv_, idle_cv_;
  std::deque<Task*> queue_;
  size_t busy_ = 0;
  bool stop_ = false;
  std::mutex err_mutex_;
  std::string async_error_;
  struct Timed {
    std::string name;
    void* start;
    void* stop;
  };
  bool profile_ = false;
  std::string profile_filter_;
  std::mutex prof_mutex_;
  std::vector<Timed> timed_;
};

}  // namespace minerva
