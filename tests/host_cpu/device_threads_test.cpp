// CPU test of the GPU-independent half of the host layer: PooledDataStore and ThreadedDevice
// (thread pool, task execution, completion listener, error path) with malloc / free as the
// allocator and operators that compute on the CPU.  Built and run by tests/test_host_cpu.py
// under -fsanitize=address,undefined and under -fsanitize=thread: four worker threads plus
// two producer threads push, run and free tasks concurrently, which is how the engine's
// dispatcher threads drive a device (reference minerva/device/device.cpp:52-119,
// pooled_data_store.cpp:19-65).  Prints "OK" and exits 0 when every check holds.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>

#include "device.h"

using namespace minerva;

#define REQUIRE(cond)                                                        \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::fprintf(stderr, "%s:%d: failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                          \
    }                                                                        \
  } while (0)

namespace {

std::atomic<long> g_allocs{0}, g_frees{0};
void* CountingAlloc(size_t n) {
  ++g_allocs;
  return std::malloc(n);
}
void CountingFree(void* p) {
  ++g_frees;
  std::free(p);
}

class FillFn : public ComputeFn {
 public:
  explicit FillFn(float v) : v_(v) {}
  void Execute(const DataList&, const DataList& out, const Context&) override {
    for (int i = 0; i < out[0].size_.Prod(); ++i) out[0].data_[i] = v_ + i;
  }
  std::string Name() const override { return "fill"; }

 private:
  float v_;
};

class AddFn : public ComputeFn {
 public:
  void Execute(const DataList& in, const DataList& out, const Context&) override {
    for (int i = 0; i < out[0].size_.Prod(); ++i) out[0].data_[i] = in[0].data_[i] + in[1].data_[i];
  }
  std::string Name() const override { return "+"; }
};

class ThrowFn : public ComputeFn {
 public:
  void Execute(const DataList&, const DataList&, const Context&) override {
    MNV_FATAL() << "operator failed on purpose";
  }
  std::string Name() const override { return "throw"; }
};

class MallocDevice : public ThreadedDevice {
 public:
  MallocDevice(uint64_t id, DeviceListener* l, size_t threshold) : ThreadedDevice(id, l, 4) {
    data_store_.reset(new PooledDataStore(threshold, CountingAlloc, CountingFree));
  }
  ~MallocDevice() override { StopWorkers(); }
  std::string Name() const override { return "malloc device"; }
  MemType GetMemType() const override { return MemType::kCpu; }
  PooledDataStore& store() { return *data_store_; }
  std::atomic<int> pre_executes{0};

 protected:
  void PreExecute() override { ++pre_executes; }
  void DoCopyRemoteData(float* dst, float* src, size_t bytes, int) override {
    std::memcpy(dst, src, bytes);
  }
  void DoExecute(const DataList& in, const DataList& out, PhysicalOp& op, int) override {
    Context ctx;
    ctx.impl_type = ImplType::kBasic;
    op.compute_fn->Execute(in, out, ctx);
  }
};

struct Counter : DeviceListener {
  std::atomic<long> done{0};
  void OnOperationComplete(Task*) override { ++done; }
};

Task MakeTask(uint64_t dev, std::shared_ptr<ComputeFn> fn, std::vector<uint64_t> in, uint64_t out,
              const Scale& size, bool light) {
  Task t;
  for (auto id : in) t.inputs.emplace_back(PhysicalData(size, dev, id), id);
  t.outputs.emplace_back(PhysicalData(size, dev, out), out);
  t.op.compute_fn = std::move(fn);
  t.light = light;
  return t;
}

void TestStorePolicy() {
  g_allocs = g_frees = 0;
  {
    PooledDataStore store(1000, CountingAlloc, CountingFree);
    float* a = store.CreateData(1, 400);
    REQUIRE(store.ExistData(1) && store.GetData(1) == a && store.GetTotalBytes() == 400);
    store.FreeData(1);
    REQUIRE(!store.ExistData(1) && store.NumCachedBlocks() == 1 && store.GetTotalBytes() == 400);
    REQUIRE(store.CreateData(2, 400) == a);                 // exact size: served from the list
    REQUIRE(g_allocs == 1);
    float* b = store.CreateData(3, 404);                    // another size: a new block
    REQUIRE(b != a && g_allocs == 2 && store.GetTotalBytes() == 804);
    store.FreeData(3);
    store.CreateData(4, 300);                               // 1104 > 1000: cached blocks dropped
    REQUIRE(store.NumCachedBlocks() == 0 && g_frees == 1 && store.GetTotalBytes() == 700);
    bool threw = false;
    try {
      store.CreateData(4, 8);
    } catch (const Error&) {
      threw = true;
    }
    REQUIRE(threw);                                         // duplicate id
    try {
      threw = false;
      store.GetData(99);
    } catch (const Error&) {
      threw = true;
    }
    REQUIRE(threw);
    // stream-aware recycling: a block another stream still uses is avoided below half the
    // threshold and handed out with the streams to wait for above it
    PooledDataStore df(4000, CountingAlloc, CountingFree);
    float* p = df.CreateData(1, 256, 0);
    df.FreeData(1, 1u << 0 | 1u << 2);                      // streams 0 and 2 have work on it
    unsigned foreign = 7;
    float* q = df.CreateData(2, 256, 1, &foreign);
    REQUIRE(q != p && foreign == 0);                        // a fresh block, nothing to wait for
    df.FreeData(2, 1u << 1);
    REQUIRE(df.CreateData(3, 256, 1, &foreign) == q && foreign == 0);   // its own block again
    df.CreateData(10, 1800, 1);                             // past half the threshold now
    float* r = df.CreateData(4, 256, 3, &foreign);
    REQUIRE(r == p && foreign == (1u << 0 | 1u << 2));      // recycled, with the streams to wait for
    df.FreeData(4, 1u << 3);
    df.ClearUsers();
    REQUIRE(df.CreateData(5, 256, 0, &foreign) == p && foreign == 0);
  }
  REQUIRE(g_allocs == g_frees);                             // the destructor returns everything
}

void TestConcurrentStore() {
  PooledDataStore store(1 << 20, CountingAlloc, CountingFree);
  std::vector<std::thread> ts;
  for (int t = 0; t < 4; ++t)
    ts.emplace_back([&store, t] {
      for (int i = 0; i < 3000; ++i) {
        uint64_t id = (uint64_t)t << 32 | (uint64_t)i;
        size_t bytes = 64 * (1 + i % 7);
        float* p = store.CreateData(id, bytes);
        p[0] = (float)i;
        REQUIRE(store.GetData(id) == p && p[0] == (float)i);
        store.FreeData(id);
      }
    });
  for (auto& t : ts) t.join();
  REQUIRE(store.GetTotalBytes() <= (1u << 20) + 64 * 7);
}

void TestDevice() {
  Counter listener;
  const Scale size{257};
  const int kTasks = 600;
  {
    MallocDevice dev(7, &listener, 1 << 22);
    // two inputs created by light tasks on the caller's thread
    Task fa = MakeTask(7, std::make_shared<FillFn>(1.f), {}, 1, size, true);
    Task fb = MakeTask(7, std::make_shared<FillFn>(100.f), {}, 2, size, true);
    dev.PushTask(&fa);
    dev.PushTask(&fb);
    REQUIRE(listener.done == 2 && dev.GetPtr(1).first == Device::MemType::kCpu);
    // two producers push independent additions to the pool while freeing earlier results
    std::vector<Task> tasks;
    tasks.reserve(2 * kTasks);
    for (int i = 0; i < 2 * kTasks; ++i)
      tasks.push_back(MakeTask(7, std::make_shared<AddFn>(), {1, 2}, 1000 + i, size, false));
    auto producer = [&](int first) {
      for (int i = first; i < first + kTasks; ++i) dev.PushTask(&tasks[i]);
    };
    std::thread p0(producer, 0), p1(producer, kTasks);
    p0.join();
    p1.join();
    dev.WaitForAllFinished();
    REQUIRE(listener.done == 2 + 2 * kTasks && dev.TakeAsyncError().empty());
    REQUIRE(dev.pre_executes == 2 + 2 * kTasks);
    for (int i = 0; i < 2 * kTasks; ++i) {
      float* r = dev.GetPtr(1000 + i).second;
      for (int j = 0; j < 257; ++j) REQUIRE(r[j] == (1.f + j) + (100.f + j));
    }
    // frees race with a second wave of tasks that reuse the freed blocks
    std::thread freer([&] {
      for (int i = 0; i < 2 * kTasks; ++i) dev.FreeDataIfExist(1000 + i);
    });
    std::vector<Task> wave;
    wave.reserve(kTasks);
    for (int i = 0; i < kTasks; ++i)
      wave.push_back(MakeTask(7, std::make_shared<AddFn>(), {1, 2}, 5000 + i, size, false));
    for (auto& t : wave) dev.PushTask(&t);
    freer.join();
    dev.WaitForAllFinished();
    for (int i = 0; i < kTasks; ++i) REQUIRE(dev.GetPtr(5000 + i).second[3] == 4.f + 103.f);
    dev.FreeDataIfExist(424242);  // unknown id: a no-op, as in the reference
    REQUIRE(dev.GetMemUsage().find("device #7 used") == 0);
    // error path: the operator throws on a pool thread; the device keeps working
    long before = listener.done;
    Task bad = MakeTask(7, std::make_shared<ThrowFn>(), {1}, 9000, size, false);
    dev.PushTask(&bad);
    dev.WaitForAllFinished();
    REQUIRE(listener.done == before + 1);
    REQUIRE(dev.TakeAsyncError().find("on purpose") != std::string::npos);
    Task missing = MakeTask(7, std::make_shared<AddFn>(), {1, 777}, 9001, size, true);
    bool threw = false;
    try {
      dev.PushTask(&missing);  // light task: the failed check surfaces on the caller's thread
    } catch (const Error&) {
      threw = true;
    }
    REQUIRE(threw);
    Task remote = MakeTask(8, std::make_shared<AddFn>(), {1, 2}, 9002, size, true);
    remote.inputs[0].physical_data.device_id = 8;
    threw = false;
    try {
      dev.PushTask(&remote);
    } catch (const Error&) {
      threw = true;
    }
    REQUIRE(threw);
    Task ok = MakeTask(7, std::make_shared<AddFn>(), {1, 2}, 9003, size, false);
    dev.PushTask(&ok);
    dev.WaitForAllFinished();
    REQUIRE(dev.GetPtr(9003).second[0] == 101.f && dev.TakeAsyncError().empty());
  }
  REQUIRE(g_allocs == g_frees);
}

}  // namespace

int main() {
  TestStorePolicy();
  TestConcurrentStore();
  g_allocs = g_frees = 0;
  TestDevice();
  std::printf("OK\n");
  return 0;
}
