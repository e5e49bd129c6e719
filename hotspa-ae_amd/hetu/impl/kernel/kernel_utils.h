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
