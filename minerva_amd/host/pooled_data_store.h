// The device allocator: exact-size free lists over an allocator / deallocator pair, the
// policy of the reference's PooledDataStore (minerva/device/pooled_data_store.cpp:19-65):
// a freed block is cached under its byte size and handed to the next request of exactly that
// size; when the bytes held exceed the threshold every cached block is released.  The
// allocator functors make it independent of the GPU (hipMalloc / hipFree on the device,
// malloc / free in the CPU tests of the host layer).
// Added for the dataflow mode of the HIP device: a cached block remembers which streams still
// have work queued on it, so that a request from another stream can avoid it or wait.
#pragma once
#include <cstddef>
#include <cstdint>
#include <deque>
#include <functional>
#include <mutex>
#include <unordered_map>

namespace minerva {

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

}  // namespace minerva
