// NDArray: reference-counted handle to {meta, storage, storage offset}; the type
// every kernel entry point takes (hetu/core/ndarray.h:17-25, 590-780 of the
// reference).  Only what the row-wise operator path needs is here: creation,
// views, host/device copies, MarkUsedBy and the operator statics that dispatch
// to LayerNorm / FusedLayerNorm / Softmax / SoftmaxCrossEntropy(Sparse) / Reduce.
#pragma once

#include <memory>
#include <ostream>
#include <vector>

#include "hetu/core/memory_pool.h"
#include "hetu/core/ndarray_meta.h"
#include "hetu/core/ndarray_storage.h"
#include "hetu/core/reduction_type.h"
#include "hetu/core/stream.h"

namespace hetu {

class NDArrayDef;
class NDArray;
using NDArrayList = std::vector<NDArray>;

class NDArrayDef {
 public:
  NDArrayDef(const NDArrayMeta& meta, std::shared_ptr<NDArrayStorage> storage, int64_t storage_offset = 0)
  : _meta(meta), _storage(std::move(storage)), _storage_offset(storage_offset) {
    HT_ASSERT(_meta.dtype != kUndeterminedDataType && !_meta.device.is_undetermined())
      << "Invalid meta: " << _meta;
    HT_VALUE_ERROR_IF(_storage == nullptr) << "Storage is not provided";
    HT_ASSERT_GE(storage_offset, 0) << "Storage offset should be greater or equal to 0";
    HT_ASSERT_GE(_storage->size(), min_storage_size(storage_offset)) << "Storage size is not sufficient";
  }
  NDArrayDef(const NDArrayDef&) = delete;
  NDArrayDef& operator=(const NDArrayDef&) = delete;

  void* raw_data_ptr() {
    return static_cast<uint8_t*>(_storage->mutable_data()) + _storage_offset * DataType2Size(dtype());
  }
  const void* raw_data_ptr() const {
    return static_cast<const uint8_t*>(_storage->data()) + _storage_offset * DataType2Size(dtype());
  }
  template <typename T> T* data_ptr() { return static_cast<T*>(raw_data_ptr()); }
  template <typename T> const T* data_ptr() const { return static_cast<const T*>(raw_data_ptr()); }

  const NDArrayMeta& meta() const { return _meta; }
  size_t ndim() const { return _meta.ndim(); }
  size_t numel() const { return _meta.numel(); }
  DataType dtype() const { return _meta.dtype; }
  Device device() const { return _meta.device; }
  bool is_cpu() const { return _meta.device.is_cpu(); }
  bool is_cuda() const { return _meta.device.is_cuda(); }
  const HTShape& shape() const { return _meta.shape; }
  int64_t shape(size_t axis) const { return _meta.shape.at(axis); }
  const HTStride& stride() const { return _meta.stride; }
  int64_t stride(int64_t axis) const {
    const int64_t nd = static_cast<int64_t>(ndim());
    HT_ASSERT(axis >= -nd && axis < nd) << "stride should in range [" << -nd << "," << nd << "), but it's " << axis;
    return _meta.stride[axis < 0 ? axis + nd : axis];
  }
  bool is_contiguous() const { return _meta.is_contiguous(); }
  const std::shared_ptr<NDArrayStorage>& storage() const { return _storage; }
  size_t storage_size() const { return _storage->size(); }
  int64_t storage_offset() const { return _storage_offset; }
  size_t min_storage_size(int64_t storage_offset) const {
    // the last addressed element of a (possibly strided) view
    int64_t span = 1;
    for (size_t i = 0; i < ndim(); ++i) {
      if (shape(i) == 0) return size_t(storage_offset) * DataType2Size(dtype());
      span += (shape(i) - 1) * _meta.stride[i];
    }
    return size_t(storage_offset + span) * DataType2Size(dtype());
  }
  void wait() const;   // blocks the host until every stream that used the storage is done

 private:
  NDArrayMeta _meta;
  std::shared_ptr<NDArrayStorage> _storage;
  int64_t _storage_offset;
};

class NDArray {
 public:
  NDArray() = default;
  NDArray(const NDArrayMeta& meta, std::shared_ptr<NDArrayStorage> storage, int64_t storage_offset = 0)
  : _ptr(std::make_shared<NDArrayDef>(meta, std::move(storage), storage_offset)) {}

  bool is_defined() const { return _ptr != nullptr; }
  NDArrayDef* operator->() const { return _ptr.get(); }
  NDArrayDef& operator*() const { return *_ptr; }
  bool operator==(const NDArray& o) const { return _ptr == o._ptr; }

  static const StreamIndex DEFAULT_STREAM;

  // Tells the allocator that `stream` has work queued on the storage, so the
  // block is not handed to another stream before that work is done.
  static void MarkUsedBy(const NDArray& array, const Stream& stream);
  static void MarkUsedBy(const NDArrayList& arrays, const Stream& stream);

  static NDArray empty(const HTShape& shape, const Device& device = Device(kCPU), DataType dtype = kFloat32,
                       StreamIndex stream_id = DEFAULT_STREAM);
  static NDArray empty_like(const NDArray& other, StreamIndex stream_id = DEFAULT_STREAM);
  static NDArray zeros(const HTShape& shape, const Device& device = Device(kCPU), DataType dtype = kFloat32,
                       StreamIndex stream_id = DEFAULT_STREAM);
  static NDArray zeros_like(const NDArray& other, StreamIndex stream_id = DEFAULT_STREAM);
  // Wraps memory owned by someone else (no copy, never freed by the pool).
  static NDArray borrow(void* ptr, const HTShape& shape, const Device& device, DataType dtype,
                        const HTStride& stride = {});
  static NDArray view(const NDArray& input, const HTShape& view_shape);   // one extent may be -1
  static NDArray as_strided(const NDArray& input, const HTShape& shape, const HTStride& stride,
                            int64_t storage_offset = 0);
  static NDArray permute(const NDArray& input, const HTAxes& dims);
  static NDArray slice(const NDArray& input, const HTShape& begin_pos, const HTShape& shape);
  static NDArray contiguous(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM);
  // device <-> host copies of contiguous arrays (no dtype conversion)
  static NDArray to(const NDArray& input, const Device& device, StreamIndex stream_id = DEFAULT_STREAM);
  static NDArray cuda(const NDArray& input, DeviceIndex dev_id = 0, StreamIndex stream_id = DEFAULT_STREAM) {
    return to(input, Device(kCUDA, dev_id), stream_id);
  }
  static NDArray cpu(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM) {
    return to(input, Device(kCPU), stream_id);
  }

  // ---- operators of the row-wise path (hetu/core/ndarray.cc:433-445,
  //      1063-1087, 1148-1172, 1407-1474 of the reference) ----
  static NDArray reduce(const NDArray& input, ReductionType red_type, const HTAxes& axes = HTAxes(),
                        bool keepdims = false, StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);
  static NDArray sum(const NDArray& input, const HTAxes& axes = HTAxes(), bool keepdims = false,
                     StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY) {
    return reduce(input, kSUM, axes, keepdims, stream_id, output);
  }
  static NDArray mean(const NDArray& input, const HTAxes& axes = HTAxes(), bool keepdims = false,
                      StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY) {
    return reduce(input, kMEAN, axes, keepdims, stream_id, output);
  }
  static NDArray max(const NDArray& input, const HTAxes& axes = HTAxes(), bool keepdims = false,
                     StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY) {
    return reduce(input, kMAX, axes, keepdims, stream_id, output);
  }
  static NDArray min(const NDArray& input, const HTAxes& axes = HTAxes(), bool keepdims = false,
                     StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY) {
    return reduce(input, kMIN, axes, keepdims, stream_id, output);
  }
  static NDArray prod(const NDArray& input, const HTAxes& axes = HTAxes(), bool keepdims = false,
                      StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY) {
    return reduce(input, kPROD, axes, keepdims, stream_id, output);
  }
  static NDArrayList layernorm(const NDArray& input, const NDArray& bn_scale, const NDArray& bn_bias,
                               const HTShape& normalized_shape, double eps = 0.01,
                               StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY,
                               NDArray& save_mean = EMPTY, NDArray& save_var = EMPTY);
  static NDArrayList fused_layernorm(const NDArray& input, const NDArray& bn_scale, const NDArray& bn_bias,
                                     const HTShape& normalized_shape, double eps = 0.01,
                                     StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY,
                                     NDArray& save_mean = EMPTY, NDArray& save_var = EMPTY);
  // element-wise arithmetic with broadcasting (hetu/core/ndarray.cc:186-303, 388-404 of the reference);
  // `output` may be one of the operands of the result's shape (in place)
  static NDArray add(const NDArray& x, const NDArray& y, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray add(const NDArray& input, double scalar, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray sub(const NDArray& x, const NDArray& y, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray sub(const NDArray& input, double scalar, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray sub(double scalar, const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray neg(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);
  static NDArray mul(const NDArray& x, const NDArray& y, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray mul(const NDArray& input, double scalar, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray div(const NDArray& x, const NDArray& y, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray div(const NDArray& input, double scalar, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray div(double scalar, const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM,
                     NDArray& output = EMPTY);
  static NDArray sqrt(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);
  static NDArray exp(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);
  static NDArray log(const NDArray& input, StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);

  // p-norm over one dimension (hetu/core/ndarray.cc:1259-1279 of the reference)
  static NDArray norm(const NDArray& input, int64_t p = 1, int64_t dim = 0, bool keepdim = false,
                      StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);

  static NDArray softmax(const NDArray& input, int64_t dim, StreamIndex stream_id = DEFAULT_STREAM,
                         NDArray& output = EMPTY);
  static NDArray sceloss(const NDArray& preds, const NDArray& labels, ReductionType reduction = kMEAN,
                         StreamIndex stream_id = DEFAULT_STREAM, NDArray& output = EMPTY);
  static NDArray sceloss(const NDArray& preds, const NDArray& labels, const int64_t ignored_index,
                         ReductionType reduction = kMEAN, StreamIndex stream_id = DEFAULT_STREAM,
                         NDArray& output = EMPTY);

 private:
  static NDArray EMPTY;
  std::shared_ptr<NDArrayDef> _ptr;
};

std::ostream& operator<<(std::ostream& os, const NDArray& a);

} // namespace hetu
