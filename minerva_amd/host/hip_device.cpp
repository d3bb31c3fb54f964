#include "hip_device.h"
#include "staged_copy.h"

#include <cstdio>
#include <cstring>

#include "mnv_hip.h"

namespace minerva {

namespace {
void Ok(int status, const char* what) {
  MNV_CHECK(status == MNV_OK) << what << ": " << mnv_error_string(status);
}
// Scratch arena per worker stream: split-k partial sums of the skinny GEMMs and of the
// convolution filter gradient (the kernels use as many k ranges as fit) and the transformed
// tiles of the 3 x 3 and 5 x 5 convolutions by minimal filtering (up to 1.2 GB for 96 -> 256
// channels under 5 x 5 filters on 27 x 27 planes at batch 256; with less those run in groups of
// images).  Allocated when a stream first runs an
// operator and kept: no operator allocates, so a recorded step never meets an allocation.
constexpr size_t kWorkspaceBytes = (size_t)1280 << 20;
// Pinned staging per worker stream: two halves, one filled by the CPU while the other is
// copied to the device.
constexpr size_t kStagingBytes = (size_t)16 << 20;
}  // namespace

// ---------------------------------------------------------------------- HipDevice

HipDevice::HipDevice(uint64_t device_id, DeviceListener* listener, int gpu_id, size_t pool_bytes)
    : ThreadedDevice(device_id, listener, kParallelism), gpu_id_(gpu_id) {
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
}

HipDevice::~HipDevice() {
  StopWorkers();  // before the streams they launch on go away
  Activate();
  for (size_t i = 0; i < kParallelism; ++i) mnv_stream_sync(streams_[i]);
  for (auto& e : latest_event_)
    if (e) mnv_event_destroy(e);
  produced_.clear();
  data_store_.reset();  // before the streams: the deallocator uses the device
  for (size_t i = 0; i < kParallelism; ++i) {
    if (workspace_[i]) mnv_free(workspace_[i]);
    if (staging_[i]) mnv_host_free(staging_[i]);
    mnv_stream_destroy(streams_[i]);
  }
}

void HipDevice::Activate() const { Ok(mnv_device_set(gpu_id_), "set device"); }

// every task re-selects the device on its thread (reference device.cpp:201-203)
void HipDevice::PreExecute() { Activate(); }

void HipDevice::DoCopyRemoteData(float* dst, float* src, size_t bytes, int thrid) {
  Ok(mnv_memcpy_d2d(dst, src, bytes, streams_[thrid]), "remote copy");
  Ok(mnv_stream_sync(streams_[thrid]), "remote copy sync");
}

std::string HipDevice::Name() const {
  char buf[64];
  snprintf(buf, sizeof(buf), "HIP device #%d", static_cast<int>(device_id_));
  return buf;
}

void HipDevice::FreeDataIfExist(uint64_t data_id) {
  size_t erased;
  unsigned users = 0;
  erased = local_data_.Erase(data_id);
  {
    std::lock_guard<std::mutex> lck(local_mutex_);
    auto it = produced_.find(data_id);
    if (it != produced_.end()) {
      // The host may be far ahead of the GPU: kernels that read or write this block can
      // still be queued on these streams when the block goes back to the pool.
      users = it->second.users;
      produced_.erase(it);
    }
  }
  if (erased == 1) data_store_->FreeData(data_id, users);
}

void HipDevice::set_dataflow(bool v) {
  WaitForAllFinished();
  Activate();
  for (size_t i = 0; i < kParallelism; ++i) Ok(mnv_stream_sync(streams_[i]), "mode change sync");
  dataflow_ = v;
  if (v) sync_each_op_ = false;
}

// An event on `stream` that was recorded after operator number `seq` of that stream was
// queued.  A replaced event is destroyed; waits already queued on it keep their meaning.
void* HipDevice::EventCovering(int stream, uint64_t seq) {
  if (latest_event_[stream] && latest_event_seq_[stream] >= seq) return latest_event_[stream];
  void* e = nullptr;
  Ok(mnv_event_create_ordering(&e), "event create");
  Ok(mnv_event_record(e, streams_[stream]), "event record");
  if (latest_event_[stream]) mnv_event_destroy(latest_event_[stream]);
  latest_event_[stream] = e;
  latest_event_seq_[stream] = queued_ops_[stream];
  return e;
}

// Makes stream `thrid` wait for everything queued so far on each of `streams`.
void HipDevice::WaitForStreams(int thrid, unsigned streams) {
  for (size_t s = 0; s < kParallelism; ++s) {
    if (!(streams >> s & 1u) || static_cast<int>(s) == thrid) continue;
    void* e = nullptr;
    Ok(mnv_event_create_ordering(&e), "event create");
    Ok(mnv_event_record(e, streams_[s]), "event record");
    Ok(mnv_stream_wait_event(streams_[thrid], e), "stream wait");
    mnv_event_destroy(e);
    ++recycle_waits_;
  }
}

void HipDevice::PushTask(Task* task) {
  if (task->light) {  // light tasks skip the thread hop (device.cpp:55-61)
    MNV_CHECK(task->stream >= 0 && task->stream < static_cast<int>(kParallelism)) << "bad stream";
    MNV_CHECK(task->stream == 0 || dataflow_) << "streams other than 0 need dataflow mode";
    Execute(task, task->stream);
    return;
  }
  ThreadedDevice::PushTask(task);
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

void HipDevice::EnsureStaging(int thrid) {
  if (staging_[thrid]) return;
  Ok(mnv_host_malloc(&staging_[thrid], kStagingBytes), "pinned staging");
}

// ThreadedDevice::Execute plus what dataflow mode needs: waits for producers on other
// streams, stream-aware block recycling, and an event behind every output.
void HipDevice::Execute(Task* task, int thrid) {
  PreExecute();
  DataList input_shards;
  for (auto& i : task->inputs) {
    auto& d = i.physical_data;
    // One GPU: every input is local.  A remote input would be copied here with
    // mnv_memcpy_d2d over xGMI, as DoCopyRemoteData does in the reference.
    MNV_CHECK_EQ(d.device_id, device_id_) << "remote inputs are not part of the one-GPU build";
    MNV_CHECK_EQ(local_data_.Count(d.data_id), 1u) << "input data #" << d.data_id << " missing";
    if (dataflow_) {
      std::lock_guard<std::mutex> lck(local_mutex_);
      auto it = produced_.find(d.data_id);
      if (it != produced_.end()) {
        // produced on another stream: this stream waits for the producer on the GPU
        if (it->second.stream != thrid) {
          Ok(mnv_stream_wait_event(streams_[thrid], EventCovering(it->second.stream, it->second.seq)),
             "stream wait");
          ++producer_waits_;
        }
        it->second.users |= 1u << thrid;
      } else {
        // Created before dataflow mode was switched on (the switch drained every stream, so
        // the contents are complete): no producer to wait for, but this reader must be on
        // record, or the block could go back to the pool and on to another stream while
        // this stream's kernels still read it.
        produced_[d.data_id] = Produced{0, thrid, 1u << thrid};
      }
    }
    input_shards.emplace_back(data_store_->GetData(d.data_id), d.size);
  }
  DataList output_shards;
  for (auto& o : task->outputs) {
    size_t bytes = static_cast<size_t>(o.physical_data.size.Prod()) * sizeof(float);
    unsigned foreign = 0;
    float* ptr = data_store_->CreateData(o.physical_data.data_id, bytes, dataflow_ ? thrid : -1,
                                         &foreign);
    // a recycled block that work queued on other streams may still touch
    if (foreign) WaitForStreams(thrid, foreign);
    MNV_CHECK(local_data_.Insert(o.physical_data.data_id)) << "duplicate data";
    output_shards.emplace_back(ptr, o.physical_data.size);
  }
  MNV_CHECK(task->op.compute_fn) << "task without an operator";
  DoExecute(input_shards, output_shards, task->op, thrid);
  if (dataflow_) {
    // an operator that fills one of its inputs (LRNForward's scale) is that datum's producer
    // from now on: later readers on other streams must wait for this operator, not for the
    // one that created the block
    // The operator's kernels are queued: count it now, so that an event said to cover
    // this number was recorded behind them.
    std::lock_guard<std::mutex> lck(local_mutex_);
    const uint64_t seq = ++queued_ops_[thrid];
    const int mutated = task->op.compute_fn->MutatedInput();
    if (mutated >= 0 && mutated < static_cast<int>(task->inputs.size())) {
      auto& p = produced_[task->inputs[mutated].physical_data.data_id];
      p.seq = seq;
      p.stream = thrid;
      p.users |= 1u << thrid;
    }
    for (auto& o : task->outputs) produced_[o.physical_data.data_id] = Produced{seq, thrid, 1u << thrid};
  }
  if (listener_) listener_->OnOperationComplete(task);
}

void HipDevice::DoExecute(const DataList& in, const DataList& out, PhysicalOp& op, int thrid) {
  const bool pooled = OnPoolThread();
  EnsureWorkspace(thrid, kWorkspaceBytes);
  Context ctx;
  ctx.impl_type = ImplType::kHip;
  ctx.stream = streams_[thrid];
  ctx.workspace = workspace_[thrid];
  ctx.workspace_bytes = workspace_bytes_[thrid];
  if (!capturing_) {
    EnsureStaging(thrid);
    ctx.staging = staging_[thrid];
    ctx.staging_bytes = kStagingBytes;
  }
  Timed t{std::string(), nullptr, nullptr};
  bool timed = profile_ && !capturing_;
  if (timed) {
    t.name = op.compute_fn->Name();
    timed = profile_filter_.empty() || t.name.find(profile_filter_) != std::string::npos;
  }
  if (timed) {
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
  // A task of the thread pool runs on whichever worker took it: outside dataflow mode nothing
  // orders the four worker streams among themselves, so such a task is complete only once
  // its stream has drained (what the reference does for every task, device.cpp:221).
  if ((sync_each_op_ || (pooled && !dataflow_)) && !capturing_) {
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
  MNV_CHECK(!dataflow_) << "recording needs the one-stream order, not dataflow mode";
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
  if (dataflow_) {
    Activate();
    for (size_t i = 0; i < kParallelism; ++i) Ok(mnv_stream_sync(streams_[i]), "barrier");
    // nothing is queued any more: every cached block may go to any stream without a wait
    data_store_->ClearUsers();
    return;
  }
  Ok(mnv_stream_sync(streams_[thrid]), "barrier");
}

void HipDevice::CopyToHost(float* dst, uint64_t data_id, size_t floats) {
  MNV_CHECK(!capturing_) << "no host copies while a graph is recorded";
  Activate();
  const char* src = reinterpret_cast<const char*>(data_store_->GetData(data_id));
  char* out = reinterpret_cast<char*>(dst);
  const size_t bytes = floats * sizeof(float), half = kStagingBytes / 2;
  if (bytes <= half) {
    Ok(mnv_memcpy_d2h(out, src, bytes, streams_[0]), "copy to host");
    Ok(mnv_stream_sync(streams_[0]), "copy to host sync");
    return;
  }
  // large results come back through the pinned staging area, the DMA engine filling one
  // half while the CPU empties the other into the caller's pageable buffer
  EnsureStaging(0);
  char* stage = static_cast<char*>(staging_[0]);
  void* filled[2] = {nullptr, nullptr};
  Ok(mnv_event_create_ordering(&filled[0]), "event create");
  Ok(mnv_event_create_ordering(&filled[1]), "event create");
  const size_t chunks = (bytes + half - 1) / half;
  auto issue = [&](size_t i) {
    const size_t off = i * half, n = bytes - off < half ? bytes - off : half;
    int rc = mnv_memcpy_d2h(stage + (i & 1) * half, src + off, n, streams_[0]);
    if (rc == MNV_OK) rc = mnv_event_record(filled[i & 1], streams_[0]);
    return rc;
  };
  int rc = issue(0);
  for (size_t i = 0; i < chunks && rc == MNV_OK; ++i) {
    if (i + 1 < chunks) rc = issue(i + 1);  // the other half is free: chunk i-1 was emptied
    if (rc == MNV_OK) rc = mnv_event_sync(filled[i & 1]);
    if (rc != MNV_OK) break;
    const size_t off = i * half, n = bytes - off < half ? bytes - off : half;
    std::memcpy(out + off, stage + (i & 1) * half, n);
  }
  mnv_stream_sync(streams_[0]);
  mnv_event_destroy(filled[0]);
  mnv_event_destroy(filled[1]);
  Ok(rc, "copy to host");
}

void HipDevice::CopyFromHost(uint64_t data_id, const float* src, size_t floats) {
  MNV_CHECK(!capturing_) << "no host copies while a graph is recorded";
  Activate();
  Ok(mnv_memcpy_h2d(data_store_->GetData(data_id), src, floats * sizeof(float), streams_[0]),
     "copy from host");
  Ok(mnv_stream_sync(streams_[0]), "copy from host sync");
}

void HipDevice::CopyFromHostOn(int thrid, uint64_t data_id, const float* src, size_t floats) {
  MNV_CHECK(!capturing_) << "no host copies while a graph is recorded";
  MNV_CHECK(thrid >= 0 && thrid < static_cast<int>(kParallelism)) << "bad stream";
  Activate();
  EnsureStaging(thrid);
  Ok(StagedHostToDevice(data_store_->GetData(data_id), src, floats * sizeof(float), streams_[thrid],
                        staging_[thrid], kStagingBytes),
     "copy from host");
}

void* HipDevice::StreamMarker(int thrid) {
  Activate();
  void* e = nullptr;
  Ok(mnv_event_create_ordering(&e), "event create");
  Ok(mnv_event_record(e, streams_[thrid]), "event record");
  return e;
}

void HipDevice::WaitMarker(void* marker) {
  if (!marker) return;
  Ok(mnv_event_sync(marker), "event sync");
  mnv_event_destroy(marker);
}

void HipDevice::CopyOnDevice(uint64_t dst_id, uint64_t src_id, size_t floats) {
  MNV_CHECK(!dataflow_) << "the in-order device copy is for the one-stream order, not dataflow mode";
  Activate();
  Ok(mnv_copy(data_store_->GetData(src_id), data_store_->GetData(dst_id), floats, streams_[0]),
     "device copy");
}

}  // namespace minerva
