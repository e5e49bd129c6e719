// Owns one allocation of a memory pool; the block goes back to the pool when the
// last NDArray sharing it dies (hetu/core/ndarray_storage.h:17-26 of the reference).
#pragma once

#include "hetu/core/memory_pool.h"

namespace hetu {

class NDArrayStorage {
 public:
  explicit NDArrayStorage(DataPtr ptr, bool in_mempool = true) : _ptr(ptr), _in_mempool(in_mempool) {}
  NDArrayStorage(const NDArrayStorage&) = delete;
  NDArrayStorage& operator=(const NDArrayStorage&) = delete;
  ~NDArrayStorage() {
    if (_in_mempool) {
      try { FreeToMemoryPool(_ptr); } catch (...) {}
    }
  }
  size_t size() const { return _ptr.size; }
  void* mutable_data() { return _ptr.ptr; }
  const void* data() const { return _ptr.ptr; }
  const Device& device() const { return _ptr.device; }
  DataPtr data_ptr() const { return _ptr; }
  bool is_new_malloc() const { return _ptr.is_new_malloc; }

 private:
  DataPtr _ptr;
  bool _in_mempool;
};

} // namespace hetu
