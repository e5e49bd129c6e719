#include "hetu/core/memory_pool.h"

#include <map>

namespace hetu {

namespace {
struct Registry {
  std::mutex mtx;
  std::map<Device, std::function<std::shared_ptr<MemoryPool>()>> ctors;
  std::map<Device, std::shared_ptr<MemoryPool>> pools;
};
Registry& registry() {
  static Registry* r = new Registry();   // never destroyed: pools outlive static NDArrays
  return *r;
}
} // namespace

void RegisterMemoryPoolCtor(const Device& device, std::function<std::shared_ptr<MemoryPool>()> ctor) {
  auto& r = registry();
  std::lock_guard<std::mutex> lock(r.mtx);
  r.ctors[device] = std::move(ctor);
}

std::shared_ptr<MemoryPool> GetMemoryPool(const Device& device) {
  auto& r = registry();
  std::lock_guard<std::mutex> lock(r.mtx);
  auto it = r.pools.find(device);
  if (it != r.pools.end()) return it->second;
  auto ct = r.ctors.find(device);
  HT_ASSERT(ct != r.ctors.end()) << "No memory pool is registered for device " << device;
  auto pool = ct->second();
  r.pools[device] = pool;
  return pool;
}

DataPtr AllocFromMemoryPool(const Device& device, size_t num_bytes, const Stream& stream) {
  return GetMemoryPool(device)->AllocDataSpace(num_bytes, stream);
}

DataPtr BorrowToMemoryPool(const Device& device, void* ptr, size_t num_bytes, DataPtrDeleter deleter) {
  return GetMemoryPool(device)->BorrowDataSpace(ptr, num_bytes, std::move(deleter));
}

void FreeToMemoryPool(DataPtr ptr) {
  if (ptr.ptr == nullptr && ptr.size == 0) return;
  GetMemoryPool(ptr.device)->FreeDataSpace(ptr);
}

} // namespace hetu
