// Shape / stride / dtype / device of an NDArray plus the shape algebra the
// row-wise operators need (hetu/core/ndarray_meta.{h,cc} of the reference).
#pragma once

#include <cstdint>
#include <ostream>
#include <vector>

#include "hetu/core/device.h"
#include "hetu/core/dtype.h"

namespace hetu {

using HTShape = std::vector<int64_t>;
using HTStride = std::vector<int64_t>;
using HTAxes = std::vector<int64_t>;
using HTShapeList = std::vector<HTShape>;
constexpr size_t HT_MAX_NDIM = 16;

inline int64_t NumEl(const HTShape& shape) {
  int64_t n = 1;
  for (auto s : shape) n *= s;
  return n;
}

inline HTStride Shape2Stride(const HTShape& shape) {
  HTStride stride(shape.size(), 1);
  for (int i = int(shape.size()) - 2; i >= 0; --i) stride[i] = stride[i + 1] * shape[i + 1];
  return stride;
}

inline std::ostream& operator<<(std::ostream& os, const std::vector<int64_t>& v) {
  os << "[";
  for (size_t i = 0; i < v.size(); ++i) os << (i ? "," : "") << v[i];
  return os << "]";
}

class NDArrayMeta {
 public:
  NDArrayMeta() = default;
  NDArrayMeta(const HTShape& shape_, DataType dtype_, const Device& device_, const HTStride& stride_ = {})
  : dtype(dtype_), device(device_) {
    set_shape(shape_);
    if (!stride_.empty()) set_stride(stride_);
  }
  bool operator==(const NDArrayMeta& m) const {
    return dtype == m.dtype && device == m.device && shape == m.shape && stride == m.stride;
  }
  bool operator!=(const NDArrayMeta& m) const { return !(*this == m); }
  size_t ndim() const { return shape.size(); }
  size_t numel() const { return static_cast<size_t>(NumEl(shape)); }
  NDArrayMeta& set_dtype(DataType t) { dtype = t; return *this; }
  NDArrayMeta& set_device(const Device& d) { device = d; return *this; }
  NDArrayMeta& set_shape(const HTShape& s) {
    HT_ASSERT(s.size() <= HT_MAX_NDIM) << "Currently we only support shape up to " << HT_MAX_NDIM << " dimensions";
    shape = s;
    stride = Shape2Stride(shape);
    return *this;
  }
  NDArrayMeta& set_stride(const HTStride& s) {
    HT_ASSERT(s.size() == shape.size()) << "Stride " << s << " does not match shape " << shape;
    stride = s;
    return *this;
  }
  bool is_contiguous() const {
    if (ndim() < 1 || numel() <= 1) return true;
    int64_t expect = 1;
    for (int i = int(ndim()) - 1; i >= 0; --i) {
      if (stride[i] != expect) return false;
      expect *= shape[i];
    }
    return true;
  }

  // axis helpers (hetu/core/ndarray_meta.cc:135-223 of the reference)
  static int64_t ParseAxis(int64_t axis, int64_t num_dim);
  static HTAxes ParseAxes(const HTAxes axes, int64_t num_dim);
  static HTShape Reduce(const HTShape& shape, const HTAxes& axes, bool keepdims);
  // shape two operands broadcast to (trailing dimensions aligned, extent 1 repeats); empty when they cannot
  // (hetu/core/ndarray_meta.cc:99-117 of the reference)
  static HTShape Broadcast(const HTShape& shape_a, const HTShape& shape_b);

  DataType dtype{kUndeterminedDataType};
  Device device;
  HTShape shape;
  HTStride stride;
};

std::ostream& operator<<(std::ostream& os, const NDArrayMeta& meta);

} // namespace hetu
