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

// The row operands of ONE kernel call on joint levels, for the *_strided_rows entry points.  A view whose leading
// dimensions are permuted (x.permute(0, 2, 1, 3): rows contiguous, leading dimensions not on one pitch) keeps its
// rows on up to three levels, row r = (i2 * n1 + i1) * n0 + i0 starting i0 * s0 + i1 * s1 + i2 * s2 elements from
// the base; the kernels take that as it is, so such an operand is read / written in place where the reference
// walks it through its OffsetCalculator (hetu/impl/utils/offset_calculator.cuh:16-68).  Leading dimensions are
// merged where they step together in EVERY operand of the call, since all operands share one numbering of the
// rows.  What does not fit (trailing dimensions that are not dense, more than three levels) falls back operand
// by operand: an input is gathered into a dense copy, an output is written dense into pool memory and laid over
// its strides by Commit().
class RowPlan {
 public:
  struct Slot {
    NDArray array;              // what the kernel reads or writes
    NDArray* target = nullptr;  // outputs: the caller's array
    int64_t steps[3] = {0, 0, 0};
    bool defined() const { return array.is_defined(); }
    void* ptr() { return array.is_defined() ? array->raw_data_ptr() : nullptr; }
    const int64_t* steps_or_null() const { return array.is_defined() ? steps : nullptr; }
    bool staged() const { return target != nullptr && array->raw_data_ptr() != (*target)->raw_data_ptr(); }
  };

  RowPlan(int64_t inner_dims, const Stream& stream) : inner_dims_(inner_dims), stream_(stream) {}

  // an undefined array is an absent optional operand
  Slot& Input(const NDArray& a) {
    slots_[count_].array = a;
    return slots_[count_++];
  }
  Slot& Output(NDArray& a) {
    slots_[count_].array = a;
    slots_[count_].target = a.is_defined() ? &a : nullptr;
    return slots_[count_++];
  }

  // call once after every operand has been added.  vector_rows_only: the kernels behind the call take several
  // levels on their 128-bit path only (softmax, cross-entropy), so rows and steps that are not whole 16-byte
  // vectors go dense as well
  void Resolve(bool vector_rows_only = false) {
    // an operand whose trailing dimensions are not dense has no 128-bit row at all
    for (int k = 0; k < count_; ++k)
      if (slots_[k].defined() && !TrailingDense(slots_[k].array)) MakeDense(slots_[k]);
    if (!JointLevels() || (vector_rows_only && level_rows_[1] * level_rows_[2] > 1 && !WholeVectors())) {
      // too many levels: everything that is not on one pitch by itself goes dense, which leaves one level
      for (int k = 0; k < count_; ++k) {
        int64_t pitch = 0;
        if (slots_[k].defined() && !RowPitch(slots_[k].array, inner_dims_, &pitch)) MakeDense(slots_[k]);
      }
      const bool ok = JointLevels();
      HT_ASSERT(ok) << "row operands do not reduce to one level";
    }
  }

  const int64_t* level_rows() const { return level_rows_; }

  // after the kernel call, on the same stream
  void Commit() {
    for (int k = 0; k < count_; ++k) {
      Slot& sl = slots_[k];
      if (!sl.defined() || !sl.staged()) continue;
      HIPStream hip_stream(stream_);
      const HTShape& shape = (*sl.target)->shape();
      const HTStride& stride = (*sl.target)->stride();
      HK_CALL(hk_strided_scatter(int((*sl.target)->dtype()), sl.array->raw_data_ptr(), (*sl.target)->raw_data_ptr(),
                                 int(shape.size()), shape.data(), stride.data(), hip_stream));
      NDArray::MarkUsedBy({sl.array, *sl.target}, stream_);
    }
  }

  // every array a kernel call touches, for NDArray::MarkUsedBy
  NDArrayList arrays() const {
    NDArrayList out;
    for (int k = 0; k < count_; ++k)
      if (slots_[k].defined()) out.push_back(slots_[k].array);
    return out;
  }

 private:
  bool TrailingDense(const NDArray& a) const {
    const int64_t nd = int64_t(a->ndim());
    int64_t expect = 1;
    for (int64_t i = nd - 1; i >= nd - inner_dims_; --i) {
      if (a->shape(i) != 1 && a->stride(i) != expect) return false;
      expect *= a->shape(i);
    }
    return true;
  }
  // every base address and every step a whole number of 16-byte vectors
  bool WholeVectors() const {
    for (int k = 0; k < count_; ++k) {
      if (!slots_[k].defined()) continue;
      const size_t es = DataType2Size(slots_[k].array->dtype());
      if (reinterpret_cast<uintptr_t>(slots_[k].array->raw_data_ptr()) % 16 != 0) return false;
      for (int j = 0; j < 3; ++j)
        if ((size_t(slots_[k].steps[j]) * es) % 16 != 0) return false;
    }
    return true;
  }
  void MakeDense(Slot& sl) {
    if (sl.target == nullptr) {
      sl.array = NDArray::contiguous(sl.array, stream_.stream_index());
    } else {
      sl.array = NDArray::empty((*sl.target)->shape(), (*sl.target)->device(), (*sl.target)->dtype(),
                                stream_.stream_index());
    }
  }
  // merges the leading dimensions over all operands; false when more than three levels remain
  bool JointLevels() {
    const Slot* ref = nullptr;
    for (int k = 0; k < count_; ++k)
      if (slots_[k].defined()) { ref = &slots_[k]; break; }
    int64_t counts[3] = {1, 1, 1};
    int64_t steps[kMaxSlots][3];
    int levels = 0;
    const int64_t nd = ref ? int64_t(ref->array->ndim()) : 0;
    int64_t cols = 1;
    for (int64_t i = nd - inner_dims_; i < nd; ++i) cols *= ref->array->shape(i);
    for (int k = 0; k < count_; ++k) { steps[k][0] = cols; steps[k][1] = steps[k][2] = 0; }
    for (int64_t i = nd - inner_dims_ - 1; i >= 0; --i) {
      const int64_t n = ref->array->shape(i);
      if (n == 1) continue;
      bool merges = levels > 0;
      for (int k = 0; k < count_ && merges; ++k)
        if (slots_[k].defined() && slots_[k].array->stride(i) != counts[levels - 1] * steps[k][levels - 1]) merges = false;
      if (merges) {
        counts[levels - 1] *= n;
        continue;
      }
      if (levels == 3) return false;
      counts[levels] = n;
      for (int k = 0; k < count_; ++k)
        if (slots_[k].defined()) steps[k][levels] = slots_[k].array->stride(i);
      ++levels;
    }
    for (int j = 0; j < 3; ++j) level_rows_[j] = counts[j];
    for (int k = 0; k < count_; ++k)
      for (int j = 0; j < 3; ++j) slots_[k].steps[j] = steps[k][j];
    return true;
  }

  static constexpr int kMaxSlots = 8;
  Slot slots_[kMaxSlots];
  int count_ = 0;
  int64_t inner_dims_;
  Stream stream_;
  int64_t level_rows_[3] = {1, 1, 1};
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
