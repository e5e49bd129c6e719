#include "hetu/core/ndarray.h"

#include <algorithm>
#include <cstring>
#include <numeric>

#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/stream/CPUStream.h"
#include "hetu/impl/stream/HIPStream.h"
#include "hetu/impl/utils/hip_utils.h"

namespace hetu {

NDArray NDArray::EMPTY;
const StreamIndex NDArray::DEFAULT_STREAM = kComputingStream;

void NDArrayDef::wait() const {
  GetMemoryPool(device())->WaitDataSpace(_storage->data_ptr(), false);
}

void NDArray::MarkUsedBy(const NDArray& array, const Stream& stream) {
  if (stream.is_blocking() || !array.is_defined()) return;
  GetMemoryPool(array->device())->MarkDataSpaceUsedByStream(array->storage()->data_ptr(), stream);
}

void NDArray::MarkUsedBy(const NDArrayList& arrays, const Stream& stream) {
  if (stream.is_blocking()) return;
  // one pool call per device involved
  std::vector<Device> devices;
  for (const auto& a : arrays)
    if (a.is_defined() && std::find(devices.begin(), devices.end(), a->device()) == devices.end())
      devices.push_back(a->device());
  for (const auto& d : devices) {
    DataPtrList ptrs;
    for (const auto& a : arrays)
      if (a.is_defined() && a->device() == d) ptrs.push_back(a->storage()->data_ptr());
    GetMemoryPool(d)->MarkDataSpacesUsedByStream(ptrs, stream);
  }
}

NDArray NDArray::empty(const HTShape& shape, const Device& device, DataType dtype, StreamIndex stream_id) {
  NDArrayMeta meta(shape, dtype, device);
  for (auto s : shape) HT_VALUE_ERROR_IF(s < 0) << "Negative extent in shape " << shape;
  auto storage = std::make_shared<NDArrayStorage>(
    AllocFromMemoryPool(device, meta.numel() * DataType2Size(dtype), Stream(device, stream_id)));
  return NDArray(meta, storage);
}

NDArray NDArray::empty_like(const NDArray& other, StreamIndex stream_id) {
  return empty(other->shape(), other->device(), other->dtype(), stream_id);
}

NDArray NDArray::zeros(const HTShape& shape, const Device& device, DataType dtype, StreamIndex stream_id) {
  NDArray out = empty(shape, device, dtype, stream_id);
  const size_t bytes = out->numel() * DataType2Size(dtype);
  if (bytes == 0) return out;
  if (device.is_cpu()) {
    std::memset(out->raw_data_ptr(), 0, bytes);
  } else {
    Stream stream(device, stream_id);
    hetu::impl::HIPStream hs(stream);
    hetu::hip::DeviceGuard guard(device.index());
    HK_CALL(hk_memset(out->raw_data_ptr(), 0, bytes, hs.handle()));
    MarkUsedBy(out, stream);
  }
  return out;
}

NDArray NDArray::zeros_like(const NDArray& other, StreamIndex stream_id) {
  return zeros(other->shape(), other->device(), other->dtype(), stream_id);
}

NDArray NDArray::borrow(void* ptr, const HTShape& shape, const Device& device, DataType dtype,
                        const HTStride& stride) {
  NDArrayMeta meta(shape, dtype, device, stride);
  int64_t span = 1;
  for (size_t i = 0; i < meta.ndim(); ++i) {
    if (meta.shape[i] == 0) { span = 0; break; }
    span += (meta.shape[i] - 1) * meta.stride[i];
  }
  auto storage = std::make_shared<NDArrayStorage>(
    BorrowToMemoryPool(device, ptr, size_t(span) * DataType2Size(dtype), [](DataPtr) {}));
  return NDArray(meta, storage);
}

NDArray NDArray::view(const NDArray& input, const HTShape& view_shape) {
  HT_ASSERT(input->is_contiguous()) << "view needs a contiguous array, got " << input->meta();
  HTShape shape = view_shape;
  int64_t known = 1, infer = -1;
  for (size_t i = 0; i < shape.size(); ++i) {
    if (shape[i] == -1) {
      HT_VALUE_ERROR_IF(infer >= 0) << "Only one extent of a view may be -1: " << view_shape;
      infer = int64_t(i);
    } else {
      known *= shape[i];
    }
  }
  const int64_t numel = int64_t(input->numel());
  if (infer >= 0) {
    HT_VALUE_ERROR_IF(known == 0 || numel % known != 0) << "Cannot view " << input->shape() << " as " << view_shape;
    shape[infer] = numel / known;
  }
  HT_VALUE_ERROR_IF(NumEl(shape) != numel) << "Cannot view " << input->shape() << " as " << view_shape;
  NDArrayMeta meta(shape, input->dtype(), input->device());
  return NDArray(meta, input->storage(), input->storage_offset());
}

NDArray NDArray::as_strided(const NDArray& input, const HTShape& shape, const HTStride& stride,
                            int64_t storage_offset) {
  NDArrayMeta meta(shape, input->dtype(), input->device(), stride);
  return NDArray(meta, input->storage(), input->storage_offset() + storage_offset);
}

NDArray NDArray::permute(const NDArray& input, const HTAxes& dims) {
  const int64_t nd = int64_t(input->ndim());
  HT_VALUE_ERROR_IF(int64_t(dims.size()) != nd) << "permute needs " << nd << " axes, got " << dims;
  HTShape shape(nd);
  HTStride stride(nd);
  std::vector<bool> seen(nd, false);
  for (int64_t i = 0; i < nd; ++i) {
    const int64_t a = NDArrayMeta::ParseAxis(dims[i], nd);
    HT_VALUE_ERROR_IF(seen[a]) << "Repeated axis in permutation " << dims;
    seen[a] = true;
    shape[i] = input->shape(a);
    stride[i] = input->stride(a);
  }
  return as_strided(input, shape, stride);
}

NDArray NDArray::slice(const NDArray& input, const HTShape& begin_pos, const HTShape& shape) {
  HT_VALUE_ERROR_IF(begin_pos.size() != input->ndim() || shape.size() != input->ndim()) << "slice rank mismatch";
  int64_t offset = 0;
  for (size_t i = 0; i < input->ndim(); ++i) {
    HT_VALUE_ERROR_IF(begin_pos[i] < 0 || begin_pos[i] + shape[i] > input->shape(i)) << "slice out of range";
    offset += begin_pos[i] * input->stride(int64_t(i));
  }
  return as_strided(input, shape, input->stride(), offset);
}

NDArray NDArray::contiguous(const NDArray& input, StreamIndex stream_id) {
  if (input->is_contiguous()) return input;
  NDArray out = empty(input->shape(), input->device(), input->dtype(), stream_id);
  if (input->numel() == 0) return out;
  if (input->is_cpu()) {
    // on the host stream, behind whatever still has to write the input
    hetu::impl::CPUStream(Stream(input->device(), stream_id)).EnqueueTask(
      [input, out]() {
        const size_t es = DataType2Size(input->dtype());
        const auto* src = static_cast<const uint8_t*>(input->raw_data_ptr());
        auto* dst = static_cast<uint8_t*>(out->raw_data_ptr());
        const int64_t n = int64_t(input->numel()), nd = int64_t(input->ndim());
        for (int64_t i = 0; i < n; ++i) {
          int64_t rem = i, off = 0;
          for (int64_t d = nd - 1; d >= 0; --d) {
            off += (rem % input->shape(d)) * input->stride(d);
            rem /= input->shape(d);
          }
          std::memcpy(dst + i * es, src + off * es, es);
        }
      },
      "Contiguous");
    return out;
  }
  HT_NOT_IMPLEMENTED_IF(input->ndim() > 8) << "contiguous supports up to 8 dimensions on the device";
  Stream stream(input->device(), stream_id);
  hetu::impl::HIPStream hs(stream);
  hetu::hip::DeviceGuard guard(input->device().index());
  HK_CALL(hk_strided_copy(int(input->dtype()), input->raw_data_ptr(), out->raw_data_ptr(), int(input->ndim()),
                          input->shape().data(), input->stride().data(), hs.handle()));
  MarkUsedBy({input, out}, stream);
  return out;
}

NDArray NDArray::to(const NDArray& input, const Device& device, StreamIndex stream_id) {
  if (device == input->device()) return input;
  NDArray src = contiguous(input, stream_id);
  // a host source may still be the output of work on the host stream of the same index
  if (src->is_cpu()) Stream(src->device(), stream_id).Sync();
  NDArray out = empty(src->shape(), device, src->dtype(), stream_id);
  const size_t bytes = src->numel() * DataType2Size(src->dtype());
  if (bytes == 0) return out;
  const Device& gpu = device.is_cuda() ? device : src->device();
  HT_NOT_IMPLEMENTED_IF(!gpu.is_cuda() || (device.is_cuda() && src->is_cuda()))
    << "copies between " << src->device() << " and " << device << " are not part of this build";
  Stream stream(gpu, stream_id);
  hetu::impl::HIPStream hs(stream);
  hetu::hip::DeviceGuard guard(gpu.index());
  if (device.is_cuda()) HK_CALL(hk_memcpy_h2d(out->raw_data_ptr(), src->raw_data_ptr(), bytes, hs.handle()));
  else HK_CALL(hk_memcpy_d2h(out->raw_data_ptr(), src->raw_data_ptr(), bytes, hs.handle()));
  // pageable host memory: finish the copy before either side can be touched
  HK_CALL(hk_stream_sync(hs.handle()));
  return out;
}

NDArray NDArray::reduce(const NDArray& input, ReductionType red_type, const HTAxes& axes, bool keepdims,
                        StreamIndex stream_id, NDArray& output) {
  auto output_shape = NDArrayMeta::Reduce(input->shape(), axes, keepdims);
  NDArray out = output.is_defined() ? output
                                    : NDArray::empty(output_shape, input->device(), input->dtype(), stream_id);
  Stream stream(input->device(), stream_id);
  HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::Reduce, input, out, axes,
                                  red_type, stream);
  return out;
}

NDArrayList NDArray::layernorm(const NDArray& input, const NDArray& bn_scale, const NDArray& bn_bias,
                               const HTShape& normalized_shape, double eps, StreamIndex stream_id,
                               NDArray& output, NDArray& save_mean, NDArray& save_var) {
  NDArray out = output.is_defined() ? output : NDArray::empty_like(input, stream_id);
  // statistics: the input shape with the normalized dims set to 1, in the data dtype
  HTShape stat_shape = input->shape();
  for (size_t i = 0; i < normalized_shape.size() && i < stat_shape.size(); ++i)
    stat_shape[stat_shape.size() - 1 - i] = 1;
  NDArray savemean = save_mean.is_defined() ? save_mean
                                            : NDArray::empty(stat_shape, input->device(), input->dtype(), stream_id);
  NDArray savevar = save_var.is_defined() ? save_var
                                          : NDArray::empty(stat_shape, input->device(), input->dtype(), stream_id);
  Stream stream(input->device(), stream_id);
  HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::LayerNorm, input, bn_scale,
                                  bn_bias, savemean, savevar, out, int64_t(normalized_shape.size()), float(eps),
                                  stream);
  return {out, savemean, savevar};
}

NDArrayList NDArray::fused_layernorm(const NDArray& input, const NDArray& bn_scale, const NDArray& bn_bias,
                                     const HTShape& normalized_shape, double eps, StreamIndex stream_id,
                                     NDArray& output, NDArray& save_mean, NDArray& save_var) {
  NDArray out = output.is_defined() ? output : NDArray::empty_like(input, stream_id);
  // statistics (mean, 1/sqrt(var+eps)) are always fp32 for the fused variant
  HTShape stat_shape = input->shape();
  for (size_t i = 0; i < normalized_shape.size() && i < stat_shape.size(); ++i)
    stat_shape[stat_shape.size() - 1 - i] = 1;
  NDArray savemean = save_mean.is_defined() ? save_mean
                                            : NDArray::empty(stat_shape, input->device(), kFloat32, stream_id);
  NDArray savevar = save_var.is_defined() ? save_var
                                          : NDArray::empty(stat_shape, input->device(), kFloat32, stream_id);
  Stream stream(input->device(), stream_id);
  HT_DISPATCH_KERNEL_CUDA_ONLY(input->device().type(), __FUNCTION__, hetu::impl::FusedLayerNorm, input, bn_scale,
                               bn_bias, savemean, savevar, out, int64_t(normalized_shape.size()), float(eps),
                               stream);
  return {out, savemean, savevar};
}

// ---- element-wise arithmetic ------------------------------------------------
#define HT_NDARRAY_BINARY(fn, Kernel)                                                                       \
  NDArray NDArray::fn(const NDArray& x, const NDArray& y, StreamIndex stream_id, NDArray& output) {         \
    auto output_shape = NDArrayMeta::Broadcast(x->shape(), y->shape());                                     \
    HT_ASSERT(!output_shape.empty())                                                                        \
      << "Shapes cannot be broadcast together: " << x->shape() << " vs. " << y->shape();                    \
    NDArray out = output.is_defined() ? output : NDArray::empty(output_shape, x->device(), x->dtype(),      \
                                                                stream_id);                                 \
    Stream stream(x->device(), stream_id);                                                                  \
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(x->device().type(), __FUNCTION__, hetu::impl::Kernel, x, y, out,        \
                                    stream);                                                                \
    return out;                                                                                             \
  }
HT_NDARRAY_BINARY(add, AddElewise)
HT_NDARRAY_BINARY(sub, SubElewise)
HT_NDARRAY_BINARY(mul, MulElewise)
HT_NDARRAY_BINARY(div, DivElewise)
#undef HT_NDARRAY_BINARY

#define HT_NDARRAY_CONST(fn, Kernel)                                                                        \
  NDArray out = output.is_defined() ? output : NDArray::empty_like(input, stream_id);                       \
  Stream stream(input->device(), stream_id);                                                                \
  HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::Kernel, input, scalar,  \
                                  out, stream);                                                             \
  return out

NDArray NDArray::add(const NDArray& input, double scalar, StreamIndex stream_id, NDArray& output) {
  HT_NDARRAY_CONST(add, AddConst);
}
NDArray NDArray::sub(const NDArray& input, double scalar, StreamIndex stream_id, NDArray& output) {
  return NDArray::add(input, -scalar, stream_id, output);
}
NDArray NDArray::sub(double scalar, const NDArray& input, StreamIndex stream_id, NDArray& output) {
  HT_NDARRAY_CONST(sub, SubConst);
}
NDArray NDArray::mul(const NDArray& input, double scalar, StreamIndex stream_id, NDArray& output) {
  HT_NDARRAY_CONST(mul, MulConst);
}
NDArray NDArray::div(const NDArray& input, double scalar, StreamIndex stream_id, NDArray& output) {
  return NDArray::mul(input, 1.0 / scalar, stream_id, output);
}
NDArray NDArray::div(double scalar, const NDArray& input, StreamIndex stream_id, NDArray& output) {
  HT_NDARRAY_CONST(div, DivConst);
}
#undef HT_NDARRAY_CONST

#define HT_NDARRAY_UNARY(fn, Kernel)                                                                        \
  NDArray NDArray::fn(const NDArray& input, StreamIndex stream_id, NDArray& output) {                       \
    NDArray out = output.is_defined() ? output : NDArray::empty_like(input, stream_id);                     \
    Stream stream(input->device(), stream_id);                                                              \
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::Kernel, input, out,   \
                                    stream);                                                                \
    return out;                                                                                             \
  }
HT_NDARRAY_UNARY(neg, Opposite)
HT_NDARRAY_UNARY(sqrt, Sqrt)
HT_NDARRAY_UNARY(exp, Exp)
HT_NDARRAY_UNARY(log, Log)
#undef HT_NDARRAY_UNARY

NDArray NDArray::norm(const NDArray& input, int64_t p, int64_t dim, bool keepdim, StreamIndex stream_id,
                      NDArray& output) {
  NDArray out;
  if (output.is_defined()) {
    out = output;
  } else {
    HTShape outshape = input->shape();
    const int64_t axi = NDArrayMeta::ParseAxis(dim, int64_t(outshape.size()));
    if (keepdim) outshape[axi] = 1;
    else outshape.erase(outshape.begin() + axi);
    out = NDArray::empty(outshape, input->device(), input->dtype(), stream_id);
  }
  Stream stream(input->device(), stream_id);
  HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::Norm, input, out, dim, p, stream);
  return out;
}

NDArray NDArray::softmax(const NDArray& input, int64_t dim, StreamIndex stream_id, NDArray& output) {
  NDArray out = output.is_defined() ? output : NDArray::empty_like(input, stream_id);
  Stream stream(input->device(), stream_id);
  HT_DISPATCH_KERNEL_CPU_AND_CUDA(input->device().type(), __FUNCTION__, hetu::impl::Softmax, input, out, dim,
                                  stream);
  return out;
}

namespace {
// out = reduction of the per-row losses; kMEAN divides by ALL rows, ignored ones
// included, because it is a plain NDArray::reduce over `unreduced`
NDArray reduce_loss(const NDArray& preds, ReductionType reduction, StreamIndex stream_id, NDArray& output,
                    const std::function<void(NDArray&, const Stream&)>& kernel) {
  HTShape output_shape(preds->shape().begin(), preds->shape().end() - 1);
  if (output_shape.empty()) output_shape = {1};
  NDArray out;
  if (output.is_defined()) out = output;
  else if (reduction != kNONE) out = NDArray::empty({1}, preds->device(), preds->dtype(), stream_id);
  else out = NDArray::empty(output_shape, preds->device(), preds->dtype(), stream_id);
  Stream stream(preds->device(), stream_id);
  NDArray unreduced = reduction == kNONE ? out
                                         : NDArray::empty(output_shape, preds->device(), preds->dtype(), stream_id);
  kernel(unreduced, stream);
  if (reduction != kNONE) NDArray::reduce(unreduced, reduction, HTAxes(), false, stream_id, out);
  return out;
}
} // namespace

NDArray NDArray::sceloss(const NDArray& preds, const NDArray& labels, ReductionType reduction,
                         StreamIndex stream_id, NDArray& output) {
  return reduce_loss(preds, reduction, stream_id, output, [&](NDArray& unreduced, const Stream& stream) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "sceloss", hetu::impl::SoftmaxCrossEntropy, preds,
                                    labels, unreduced, stream);
  });
}

NDArray NDArray::sceloss(const NDArray& preds, const NDArray& labels, const int64_t ignored_index,
                         ReductionType reduction, StreamIndex stream_id, NDArray& output) {
  return reduce_loss(preds, reduction, stream_id, output, [&](NDArray& unreduced, const Stream& stream) {
    HT_DISPATCH_KERNEL_CPU_AND_CUDA(preds->device().type(), "sceloss", hetu::impl::SoftmaxCrossEntropySparse,
                                    preds, labels, unreduced, ignored_index, stream);
  });
}

std::ostream& operator<<(std::ostream& os, const NDArray& a) {
  if (!a.is_defined()) return os << "NDArray(undefined)";
  return os << "NDArray(" << a->meta() << ", offset=" << a->storage_offset() << ")";
}

} // namespace hetu
