// The HIP device: the replacement for the reference's GpuDevice
// (minerva/device/device.h:65-78, device.cpp:129-222) as a subclass of ThreadedDevice
// (device.h), overriding the same hooks -- PreExecute, Barrier, DoCopyRemoteData, DoExecute --
// plus Execute and PushTask for what the reference does not have:
//
//  - kParallelism (4) worker threads, each with its own HIP stream and its own
//    grow-only scratch arena; a task of the pool runs on worker `thrid` and, unless the
//    device is in dataflow mode, is synchronised before completion is reported, as the
//    reference does after every operator.
//  - PooledDataStore (pooled_data_store.h) over mnv_malloc / mnv_free.
//  - Three ways to order operators: synchronise after every one (the reference);
//    leave them in flight on one stream (stream order); or "dataflow": operators run on
//    any of the four streams, every output carries an event recorded behind its producer,
//    and a consumer on another stream waits for that event on the GPU, never on the host.
#pragma once
#include <array>
#include <atomic>
#include <functional>
#include <map>
#include <unordered_map>

#include "device.h"
#include "op_dispatch.h"

namespace minerva {

class HipDevice : public ThreadedDevice {
 public:
  static constexpr size_t kParallelism = 4;
  // 288 GB of HBM: keep up to 200 GiB in the pool before dropping cached blocks.
  static constexpr size_t kDefaultPoolBytes = (size_t)200 << 30;

  HipDevice(uint64_t device_id, DeviceListener* listener, int gpu_id,
            size_t pool_bytes = kDefaultPoolBytes);
  ~HipDevice() override;

  void PushTask(Task* task) override;
  void FreeDataIfExist(uint64_t data_id) override;
  std::string Name() const override;
  MemType GetMemType() const override { return MemType::kGpu; }

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
  void Barrier(int thrid) override;
  void* stream(int thrid) const { return streams_[thrid]; }
  PooledDataStore& data_store() { return *data_store_; }
  // Host <-> device copies on worker stream 0, synchronised.
  void CopyToHost(float* dst, uint64_t data_id, size_t floats);
  // Overwrites existing data in place (its address does not change).
  void CopyFromHost(uint64_t data_id, const float* src, size_t floats);
  // The same on worker stream `thrid`, through that stream's pinned staging area, and
  // synchronised with that stream only: work queued on the other streams keeps running while
  // the caller's thread feeds the copy.  The caller vouches that nothing queued still touches
  // the data (see StreamMarker).  This is how the next batch is loaded under a running step.
  void CopyFromHostOn(int thrid, uint64_t data_id, const float* src, size_t floats);
  // A marker behind everything queued on worker stream `thrid` so far; WaitMarker blocks the
  // caller until the GPU has passed it and releases it.
  void* StreamMarker(int thrid);
  void WaitMarker(void* marker);
  // dst <- src on worker stream 0, left in flight (a kernel, so it can be recorded).
  void CopyOnDevice(uint64_t dst_id, uint64_t src_id, size_t floats);
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

 protected:
  void Execute(Task* task, int thrid) override;
  void PreExecute() override;  // selects the GPU on the calling thread
  // dst <- src (bytes) on worker stream `thrid`, synchronised: a remote input's copy
  void DoCopyRemoteData(float* dst, float* src, size_t bytes, int thrid) override;
  void DoExecute(const DataList& in, const DataList& out, PhysicalOp& op, int thrid) override;

 private:
  void Activate() const;
  void EnsureWorkspace(int thrid, size_t bytes);
  void EnsureStaging(int thrid);

  int gpu_id_;
  bool sync_each_op_ = true;
  bool capturing_ = false;
  bool dataflow_ = false;
  // dataflow mode, guarded by local_mutex_: where each datum was produced (stream and the
  // stream's operator count once the producer was queued) and which streams have work
  // queued that touches it.  No event is recorded behind an operator: most consumers run
  // on the producer's stream, and every event costs the GPU a few microseconds between two
  // kernels.  A consumer on another stream asks for an event that covers the producer
  // (EventCovering): the stream's latest event if it was recorded after the producer,
  // otherwise a new one recorded now, behind everything the stream has been given so far.
  struct Produced {
    uint64_t seq;
    int stream;
    unsigned users;
  };
  std::unordered_map<uint64_t, Produced> produced_;
  std::array<uint64_t, kParallelism> queued_ops_{};      // operators queued per stream
  std::array<void*, kParallelism> latest_event_{};       // last event recorded per stream
  std::array<uint64_t, kParallelism> latest_event_seq_{};  // queued_ops_ when it was recorded
  void* EventCovering(int stream, uint64_t seq);  // call with local_mutex_ held
  void WaitForStreams(int thrid, unsigned streams);
  std::atomic<uint64_t> producer_waits_{0}, recycle_waits_{0};
  std::array<void*, kParallelism> streams_{};
  std::array<void*, kParallelism> workspace_{};
  std::array<size_t, kParallelism> workspace_bytes_{};
  std::array<void*, kParallelism> staging_{};  // pinned host memory, allocated at first use
  std::mutex local_mutex_;  // guards produced_
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
