// NormCuda / NormGradientCuda: arguments and meaning of
// hetu/impl/kernel/Norm1.cu:99-133 and :135-186 of the reference: the p-norm of
// one dimension, (sum |x|^p)^(1/p), and its gradient.  A negative dim counts
// from the end.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <cmath>

namespace hetu {
namespace impl {

void NormCuda(const NDArray& input, NDArray& output, int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  HT_NOT_IMPLEMENTED_IF(nd > 8) << "norms of arrays with more than 8 dimensions";
  dim = NDArrayMeta::ParseAxis(dim, nd);
  size_t kept = 1;
  for (int64_t i = 0; i < nd; ++i)
    if (i != dim) kept *= size_t(input->shape(i));
  HT_ASSERT(output->numel() == kept) << "output " << output->shape() << " does not hold the " << kept
                                     << " norms of " << input->shape() << " over dimension " << dim;
  if (kept == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  size_t ws_bytes = 0;
  HK_CALL(hk_reduce_workspace_bytes(int(input->dtype()), int(nd), input->shape().data(), input->stride().data(), 1,
                                    &dim, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, input->device(), stream);
  HK_CALL(hk_norm(int(input->dtype()), input->raw_data_ptr(), output->raw_data_ptr(), int(nd), input->shape().data(),
                  input->stride().data(), dim, p, MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({input, output, ws}, stream);
}

void NormGradientCuda(const NDArray& input, const NDArray& output, const NDArray& output_grad, NDArray& input_grad,
                      int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DEVICE(input, output_grad);
  HT_ASSERT_SAME_DEVICE(input, input_grad);
  HT_ASSERT_SAME_SHAPE(input, input_grad);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output_grad);
  HT_ASSERT_SAME_DTYPE(input, input_grad);
  HT_ASSERT_CONTIGUOUS(input_grad);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  dim = NDArrayMeta::ParseAxis(dim, nd);
  int64_t before = 1, after = 1;
  for (int64_t i = 0; i < nd; ++i) {
    if (i < dim) before *= input->shape(i);
    else if (i > dim) after *= input->shape(i);
  }
  const int64_t reduce_size = input->shape(dim);
  HT_ASSERT(int64_t(output->numel()) == before * after && int64_t(output_grad->numel()) == before * after)
    << "norm " << output->shape() << " and its gradient " << output_grad->shape() << " must hold " << before * after
    << " values for " << input->shape() << " over dimension " << dim;
  if (input->numel() == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  NDArray x = Dense(input, stream), n = Dense(output, stream), g = Dense(output_grad, stream);
  HK_CALL(hk_norm_bwd(int(input->dtype()), x->raw_data_ptr(), n->raw_data_ptr(), g->raw_data_ptr(),
                      input_grad->raw_data_ptr(), before, reduce_size, after, p, hip_stream));
  NDArray::MarkUsedBy({x, n, g, input_grad}, stream);
}

// Host twins (hetu/impl/kernel/Norm.cc of the reference): the array is seen as [before, reduce, after]; each of
// the before * after norms is a blocked sum of |x|^p in the arithmetic type, and the gradient follows the
// accelerator's three cases (p = 1: sign(x) g; p = 2: g x / n; p > 2: x |x|^(p-2) g / n^(p-1); 0 where n = 0).
namespace {
template <typename A>
inline A AbsPow(A v, int64_t p) {
  const A a = std::fabs(v);
  if (p == 1) return a;
  if (p == 2) return a * a;
  return std::pow(a, A(p));
}
} // namespace

void NormCpu(const NDArray& input, NDArray& output, int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_CONTIGUOUS(output);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  dim = NDArrayMeta::ParseAxis(dim, nd);
  int64_t before = 1, after = 1;
  for (int64_t i = 0; i < nd; ++i) {
    if (i < dim) before *= input->shape(i);
    else if (i > dim) after *= input->shape(i);
  }
  const int64_t reduce_size = input->shape(dim);
  HT_ASSERT(int64_t(output->numel()) == before * after)
    << "output " << output->shape() << " does not hold the " << before * after << " norms of " << input->shape()
    << " over dimension " << dim;
  if (before * after == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input->dtype(), spec_t, "NormCpu", [&]() {
    cpu::on_stream(stream, "NormCpu", [=]() {
      NDArray x = Dense(input, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* px = x->data_ptr<spec_t>();
      spec_t* po = output->data_ptr<spec_t>();
      cpu::parallel_rows(before * after, reduce_size, [&](int64_t o) {
        const spec_t* base = px + (o / after) * reduce_size * after + (o % after);
        const A sum = cpu::blocked_sum<A>(reduce_size, [&](int64_t k) {
          return AbsPow<A>(cpu::ld<spec_t, A>(base + k * after), p);
        });
        cpu::st<spec_t, A>(po + o, p == 1 ? sum : p == 2 ? std::sqrt(sum) : std::pow(sum, A(1) / A(p)));
      });
    });
  });
}

void NormGradientCpu(const NDArray& input, const NDArray& output, const NDArray& output_grad, NDArray& input_grad,
                     int64_t dim, int64_t p, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HT_ASSERT_SAME_DEVICE(input, output_grad);
  HT_ASSERT_SAME_DEVICE(input, input_grad);
  HT_ASSERT_SAME_SHAPE(input, input_grad);
  HT_ASSERT_SAME_DTYPE(input, output);
  HT_ASSERT_SAME_DTYPE(input, output_grad);
  HT_ASSERT_SAME_DTYPE(input, input_grad);
  HT_ASSERT_CONTIGUOUS(input_grad);
  HT_VALUE_ERROR_IF(p < 1) << "The norm's exponent must be at least 1, got " << p;
  const int64_t nd = int64_t(input->ndim());
  dim = NDArrayMeta::ParseAxis(dim, nd);
  int64_t before = 1, after = 1;
  for (int64_t i = 0; i < nd; ++i) {
    if (i < dim) before *= input->shape(i);
    else if (i > dim) after *= input->shape(i);
  }
  const int64_t reduce_size = input->shape(dim);
  HT_ASSERT(int64_t(output->numel()) == before * after && int64_t(output_grad->numel()) == before * after)
    << "norm " << output->shape() << " and its gradient " << output_grad->shape() << " must hold " << before * after
    << " values for " << input->shape() << " over dimension " << dim;
  if (input->numel() == 0) return;
  HT_DISPATCH_FLOATING_TYPES(input->dtype(), spec_t, "NormGradientCpu", [&]() {
    cpu::on_stream(stream, "NormGradientCpu", [=]() {
      NDArray x = Dense(input, stream), n = Dense(output, stream), g = Dense(output_grad, stream);
      using A = typename cpu::Arith<spec_t>::type;
      const spec_t* px = x->data_ptr<spec_t>();
      const spec_t* pn = n->data_ptr<spec_t>();
      const spec_t* pg = g->data_ptr<spec_t>();
      spec_t* pd = input_grad->data_ptr<spec_t>();
      cpu::parallel_rows(before * reduce_size, after, [&](int64_t row) {
        const int64_t b = row / reduce_size;
        for (int64_t a = 0; a < after; ++a) {
          const A v = cpu::ld<spec_t, A>(px + row * after + a);
          const A nv = cpu::ld<spec_t, A>(pn + b * after + a), gv = cpu::ld<spec_t, A>(pg + b * after + a);
          A r;
          if (p == 1) r = (v > A(0) ? A(1) : v < A(0) ? A(-1) : A(0)) * gv;
          else if (nv == A(0)) r = A(0);
          else if (p == 2) r = gv * v / nv;
          else r = v * std::pow(std::fabs(v), A(p - 2)) * gv / std::pow(nv, A(p - 1));
          cpu::st<spec_t, A>(pd + row * after + a, r);
        }
      });
    });
  });
}

} // namespace impl
} // namespace hetu
