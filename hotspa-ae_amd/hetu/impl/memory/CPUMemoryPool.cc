// Host allocations of NDArrays (hetu/impl/memory/CPUMemoryPool.{h,cc} of the
// reference): 64-byte aligned malloc, no caching.  Host arrays only stage test
// and checkpoint data on this path, so nothing here is stream-ordered:
// WaitDataSpace drains the streams that were marked.
#include <cstdlib>
#include <unordered_map>

#include "hetu/common/logging.h"
#include "hetu/core/memory_pool.h"

namespace hetu {
namespace impl {

class CPUMemoryPool final : public MemoryPool {
 public:
  CPUMemoryPool() : MemoryPool(Device(kCPU), "CPUMemPool") {}

  DataPtr AllocDataSpace(size_t num_bytes, const Stream& = Stream()) override {
    if (num_bytes == 0) return DataPtr(nullptr, 0, _device, 0);
    void* p = nullptr;
    const size_t bytes = (num_bytes + 63) / 64 * 64;
    HT_BAD_ALLOC_IF(posix_memalign(&p, 64, bytes) != 0) << "Failed to allocate " << bytes << " bytes of host memory";
    std::lock_guard<std::mutex> lock(_mtx);
    DataPtr dp(p, bytes, _device, next_id(), true);
    _entries[dp.id] = Entry{nullptr, {}};
    _allocated += bytes;
    _peak = std::max(_peak, _allocated);
    return dp;
  }

  DataPtr BorrowDataSpace(void* ptr, size_t num_bytes, DataPtrDeleter deleter, const Stream& = Stream()) override {
    HT_VALUE_ERROR_IF(ptr == nullptr && num_bytes > 0) << "Borrowing a null pointer";
    std::lock_guard<std::mutex> lock(_mtx);
    DataPtr dp(ptr, num_bytes, _device, next_id());
    _entries[dp.id] = Entry{std::move(deleter), {}, true};
    return dp;
  }

  void FreeDataSpace(DataPtr data_ptr) override {
    if (data_ptr.id == 0) return;
    Entry e;
    {
      std::lock_guard<std::mutex> lock(_mtx);
      auto it = _entries.find(data_ptr.id);
      HT_VALUE_ERROR_IF(it == _entries.end()) << "Cannot find " << data_ptr << " (freed twice?)";
      e = std::move(it->second);
      _entries.erase(it);
      if (!e.borrowed) _allocated -= data_ptr.size;
    }
    for (auto s : e.used_by) Stream::unpack(s).Sync();
    if (e.borrowed) {
      if (e.deleter) e.deleter(data_ptr);
    } else {
      std::free(data_ptr.ptr);
    }
  }

  void MarkDataSpaceUsedByStream(DataPtr data_ptr, const Stream& stream) override {
    if (data_ptr.id == 0 || !stream.is_defined() || stream.device().is_cpu()) return;
    std::lock_guard<std::mutex> lock(_mtx);
    auto it = _entries.find(data_ptr.id);
    HT_VALUE_ERROR_IF(it == _entries.end()) << "Cannot find " << data_ptr;
    auto& used = it->second.used_by;
    const auto sid = stream.pack();
    if (std::find(used.begin(), used.end(), sid) == used.end()) used.push_back(sid);
  }

  void MarkDataSpacesUsedByStream(DataPtrList& data_ptrs, const Stream& stream) override {
    for (auto& p : data_ptrs) MarkDataSpaceUsedByStream(p, stream);
  }

  std::future<void> WaitDataSpace(DataPtr data_ptr, bool async = true) override {
    std::vector<PackedStreamId> streams;
    {
      std::lock_guard<std::mutex> lock(_mtx);
      auto it = _entries.find(data_ptr.id);
      if (it != _entries.end()) streams = it->second.used_by;
    }
    auto wait = [streams]() {
      for (auto s : streams) Stream::unpack(s).Sync();
    };
    if (async) return std::async(std::launch::async, wait);
    wait();
    std::promise<void> done;
    done.set_value();
    return done.get_future();
  }

  void PrintSummary() override {
    std::lock_guard<std::mutex> lock(_mtx);
    HT_LOG_INFO << name() << ": allocated = " << _allocated << " B, peak = " << _peak << " B, live = "
                << _entries.size();
  }

 private:
  struct Entry {
    DataPtrDeleter deleter;
    std::vector<PackedStreamId> used_by;
    bool borrowed{false};
  };
  std::unordered_map<DataPtrId, Entry> _entries;
  size_t _allocated{0}, _peak{0};
};

namespace {
struct CPUMemoryPoolRegister {
  CPUMemoryPoolRegister() {
    RegisterMemoryPoolCtor(Device(kCPU), []() { return std::static_pointer_cast<MemoryPool>(std::make_shared<CPUMemoryPool>()); });
  }
};
static CPUMemoryPoolRegister cpu_memory_pool_register;
} // namespace

} // namespace impl
} // namespace hetu
