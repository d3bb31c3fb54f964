#include "pooled_data_store.h"

#include "minerva_types.h"

namespace minerva {

PooledDataStore::PooledDataStore(size_t threshold, std::function<void*(size_t)> a,
                                 std::function<void(void*)> d)
    : allocator_(std::move(a)), deallocator_(std::move(d)), threshold_(threshold) {}

PooledDataStore::~PooledDataStore() {
  for (auto& kv : data_states_) deallocator_(kv.second.ptr);
  for (auto& kv : free_space_)
    for (auto& b : kv.second) deallocator_(b.ptr);
}

float* PooledDataStore::CreateData(uint64_t id, size_t length, int stream, unsigned* foreign) {
  std::lock_guard<std::mutex> lck(access_mutex_);
  auto it = data_states_.emplace(id, DataState{nullptr, length});
  MNV_CHECK(it.second) << "data already existed";
  DataState& ds = it.first->second;
  if (foreign) *foreign = 0;
  auto hit = free_space_.find(length);
  if (hit != free_space_.end()) {  // reuse a block of exactly this size
    auto& blocks = hit->second;
    size_t pick = 0;
    bool found = stream < 0;
    if (stream >= 0) {
      // a block no other stream still works on needs no wait: stream order protects it
      const unsigned mine = 1u << stream;
      for (size_t i = 0; i < blocks.size(); ++i)
        if ((blocks[i].users & ~mine) == 0) {
          pick = i;
          found = true;
          break;
        }
      // Otherwise a new block is better than making this stream wait for the others (it
      // would wait for everything queued on them, which serialises the streams); the pool
      // grows by at most what is allocated between two synchronisations, after which
      // every cached block is free of users again.  Past half the threshold, recycle.
      if (!found && total_ + length > threshold_ / 2) {
        found = true;
        if (foreign) *foreign = blocks[0].users & ~mine;
      }
    }
    if (!found) {
      ds.ptr = allocator_(length);
      total_ += length;
      return static_cast<float*>(ds.ptr);
    }
    ds.ptr = blocks[pick].ptr;
    blocks.erase(blocks.begin() + pick);
    if (blocks.empty()) free_space_.erase(hit);
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

void PooledDataStore::FreeData(uint64_t id, unsigned users) {
  std::lock_guard<std::mutex> lck(access_mutex_);
  auto it = data_states_.find(id);
  MNV_CHECK(it != data_states_.end()) << "data #" << id << " does not exist";
  free_space_[it->second.length].push_back(FreeBlock{it->second.ptr, users});
  data_states_.erase(it);
}

void PooledDataStore::ClearUsers() {
  std::lock_guard<std::mutex> lck(access_mutex_);
  for (auto& kv : free_space_)
    for (auto& b : kv.second) b.users = 0;
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
    for (auto& b : kv.second) {
      deallocator_(b.ptr);
      total_ -= kv.first;
    }
  free_space_.clear();
}

}  // namespace minerva
