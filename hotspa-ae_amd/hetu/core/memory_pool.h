// Allocator contract behind NDArray (hetu/core/memory_pool.h:15-103 of the
// reference): a pool per device, looked up through a registry that static
// initialisers fill.
#pragma once

#include <functional>
#include <future>
#include <memory>
#include <mutex>
#include <ostream>
#include <string>
#include <vector>

#include "hetu/core/device.h"
#include "hetu/core/stream.h"

namespace hetu {

using DataPtrId = uint64_t;
using mempool_clock_t = uint64_t;

struct DataPtr {
  void* ptr{nullptr};
  size_t size{0};
  Device device;
  DataPtrId id{0};
  bool is_new_malloc{false};
  DataPtr() = default;
  DataPtr(void* p, size_t s, const Device& d, DataPtrId i, bool fresh = false)
  : ptr(p), size(s), device(d), id(i), is_new_malloc(fresh) {}
};
using DataPtrList = std::vector<DataPtr>;
using DataPtrDeleter = std::function<void(DataPtr)>;

inline std::ostream& operator<<(std::ostream& os, const DataPtr& p) {
  return os << "DataPtr(" << p.ptr << ", " << p.size << " B, " << p.device << ", id=" << p.id << ")";
}

class MemoryPool {
 public:
  MemoryPool(Device device, std::string name) : _device(device), _name(std::move(name)) {}
  virtual ~MemoryPool() = default;
  virtual DataPtr AllocDataSpace(size_t num_bytes, const Stream& stream = Stream()) = 0;
  virtual DataPtr BorrowDataSpace(void* ptr, size_t num_bytes, DataPtrDeleter deleter,
                                  const Stream& stream = Stream()) = 0;
  virtual void FreeDataSpace(DataPtr data_ptr) = 0;
  virtual void EmptyCache() {}
  virtual void MarkDataSpaceUsedByStream(DataPtr data_ptr, const Stream& stream) = 0;
  virtual void MarkDataSpacesUsedByStream(DataPtrList& data_ptrs, const Stream& stream) = 0;
  virtual std::future<void> WaitDataSpace(DataPtr data_ptr, bool async = true) = 0;
  virtual void PrintSummary() = 0;
  const Device& device() const { return _device; }
  const std::string& name() const { return _name; }

 protected:
  DataPtrId next_id() { return _next_id++; }        // caller holds _mtx
  mempool_clock_t next_clock() { return ++_clock; }  // caller holds _mtx
  const Device _device;
  const std::string _name;
  mempool_clock_t _clock{0};
  DataPtrId _next_id{1};
  std::mutex _mtx;
};

void RegisterMemoryPoolCtor(const Device& device, std::function<std::shared_ptr<MemoryPool>()> ctor);
std::shared_ptr<MemoryPool> GetMemoryPool(const Device& device);
DataPtr AllocFromMemoryPool(const Device& device, size_t num_bytes, const Stream& stream = Stream());
DataPtr BorrowToMemoryPool(const Device& device, void* ptr, size_t num_bytes, DataPtrDeleter deleter);
void FreeToMemoryPool(DataPtr ptr);

} // namespace hetu
