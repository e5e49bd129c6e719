// Shared plumbing of the kernel entry points: dense operands, pool-backed
// scratch, the rows x cols split of a normalisation.
#pragma once

#include "hetu/core/ndarray.h"
#include "hetu/impl/stream/HIPStream.h"
#include "hetu/impl/utils/hip_utils.h"
#include "hetu/impl/utils/ndarray_utils.h"

namespace hetu {
namespace impl {

// The array itself when dense, else a dense copy made on `stream`.
inline NDArray Dense(const NDArray& a, const Stream& stream) {
  if (!a.is_defined() || a->is_contiguous()) return a;
  return NDArray::contiguous(a, stream.stream_index());
}

// The [rows, cols] view the row kernels take: the last `inner_dims` dimensions hold `cols` consecutive elements
// and the leading ones step by one constant pitch (a dense array, a slice x[..., a:b] of a wider one, a
// row-padded buffer).  Sets the pitch in elements; false for any other layout (transposed, strided columns).
inline bool RowPitch(const NDArray& a, int64_t inner_dims, int64_t* pitch) {
  const int64_t nd = int64_t(a->ndim());
  const int64_t split = nd - inner_dims;
  int64_t expect = 1;
  for (int64_t i = nd - 1; i >= split; --i) {
    if (a->shape(i) != 1 && a->stride(i) != expect) return false;
    expect *= a->shape(i);
  }
  const int64_t cols = expect;
  *pitch = cols;
  bool seen = false;
  for (int64_t i = split - 1; i >= 0; --i) {
    if (a->shape(i) == 1) continue;
    if (!seen) {
      *pitch = a->stride(i);
      seen = true;
    } else if (a->stride(i) != expect) {
      return false;
    }
    expect = a->stride(i) * a->shape(i);
  }
  return *pitch >= cols;
}

// An input of a row kernel: the array itself when it is row-pitched (no copy is made), else a dense copy on
// `stream`.  This is what stands in for the reference's per-element OffsetCalculator
// (hetu/impl/utils/offset_calculator.cuh:16-68) on the operators that accept non-contiguous inputs.
inline NDArray RowOperand(const NDArray& a, int64_t inner_dims, const Stream& stream, int64_t* pitch) {
  if (a.is_defined() && RowPitch(a, inner_dims, pitch)) return a;
  NDArray dense = Dense(a, stream);
  if (dense.is_defined()) RowPitch(dense, inner_dims, pitch);
  return dense;
}

// An output of a row kernel.  A row-pitched array (dense, a column slice of a wider array, a row-padded buffer)
// is written in place.  Any other layout (a transposed view, strided columns) has no 128-bit store pattern: the
// kernel then writes a dense stand-in from the pool and Commit() lays it over the array's own strides.  The
// reference's kernels write every element through an OffsetCalculator instead
// (hetu/impl/utils/offset_calculator.cuh:16-68); here that costs one more pass, and only for such outputs.
// inner_dims < 0 asks for a dense array outright (kernels that take no pitch).
class RowOutput {
 public:
  RowOutput(NDArray& target, int64_t inner_dims, const Stream& stream) : target_(target), stream_(stream) {
    const bool in_place = inner_dims < 0 ? target->is_contiguous() : RowPitch(target, inner_dims, &pitch_);
    if (in_place) {
      work_ = target;
    } else {
      work_ = NDArray::empty(target->shape(), target->device(), target->dtype(), stream.stream_index());
      if (inner_dims >= 0) RowPitch(work_, inner_dims, &pitch_);
    }
  }
  NDArray& array() { return work_; }
  void* ptr() { return work_->raw_data_ptr(); }
  int64_t pitch() const { return pitch_; }
  bool staged() const { return work_->raw_data_ptr() != target_->raw_data_ptr(); }
  // after the kernel call, on the same stream
  void Commit() {
    if (!staged()) return;
    HIPStream hip_stream(stream_);
    const HTShape& shape = target_->shape();
    const HTStride& stride = target_->stride();
    HK_CALL(hk_strided_scatter(int(target_->dtype()), work_->raw_data_ptr(), target_->raw_data_ptr(),
                               int(shape.size()), shape.data(), stride.data(), hip_stream));
    NDArray::MarkUsedBy({work_, target_}, stream_);
  }

 private:
  NDArray& target_;
  NDArray work_;
  Stream stream_;
  int64_t pitch_ = 0;
};

inline const void* PtrOrNull(const NDArray& a) {
  return a.is_defined() ? a->raw_data_ptr() : nullptr;
}
inline void* MutPtrOrNull(NDArray& a) {
  return a.is_defined() ? a->raw_data_ptr() : nullptr;
}

// Scratch bytes from the device's memory pool, ordered on `stream`.
inline NDArray Scratch(size_t bytes, const Device& device, const Stream& stream) {
  if (bytes == 0) return NDArray();
  return NDArray::empty({int64_t(bytes)}, device, kUInt8, stream.stream_index());
}

// rows = product of the leading dims, cols = product of the last `reduce_dims`.
inline void SplitRows(const NDArray& a, int64_t reduce_dims, int64_t& rows, int64_t& cols) {
  const int64_t nd = int64_t(a->ndim());
  HT_VALUE_ERROR_IF(reduce_dims < 1 || reduce_dims > nd)
    << "Cannot normalise over " << reduce_dims << " trailing dims of " << a->shape();
  rows = cols = 1;
  for (int64_t i = 0; i < nd - reduce_dims; ++i) rows *= a->shape(i);
  for (int64_t i = nd - reduce_dims; i < nd; ++i) cols *= a->shape(i);
}

} // namespace impl
} // namespace hetu
