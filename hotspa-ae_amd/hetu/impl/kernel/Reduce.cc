// ReduceCuda / ReduceSumCuda / ReduceMeanCuda / ReduceMaxCuda / ReduceMinCuda /
// ReduceProdCuda: arguments and meaning of hetu/impl/kernel/Reduce.cu:21-59,
// ReduceSum.cu:25-42, ReduceMean.cu:35-55, ReduceMax.cu:28-41, ReduceMin.cu:28-41
// and ReduceProd.cu:26-45 of the reference.  The input may have any strides (the
// kernel plans on shape and strides); the output is written dense.
#include "hetu/graph/ops/kernel_links.h"
#include "hetu/impl/kernel/kernel_utils.h"
#include "hetu/impl/utils/cpu_utils.h"
#include "hetu/impl/utils/dispatch.h"

#include <algorithm>
#include <limits>
#include <type_traits>
#include <vector>

namespace hetu {
namespace impl {

namespace {
void LaunchReduce(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax, int op,
                  const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  const int64_t nd = int64_t(in_arr->ndim());
  HT_NOT_IMPLEMENTED_IF(nd > 8) << "reductions of arrays with more than 8 dimensions";
  size_t kept = 1;
  std::vector<bool> reduced(nd, false);
  for (int64_t i = 0; i < num_ax; ++i) {
    HT_VALUE_ERROR_IF(axes[i] < 0 || axes[i] >= nd) << "axis " << axes[i] << " out of range for " << in_arr->shape();
    reduced[axes[i]] = true;
  }
  for (int64_t i = 0; i < nd; ++i)
    if (!reduced[i]) kept *= size_t(in_arr->shape(i));
  HT_ASSERT(out_arr->numel() == kept) << "output " << out_arr->shape() << " does not hold the " << kept
                                      << " kept elements of " << in_arr->shape();
  if (kept == 0) return;

  HIPStream hip_stream(stream);
  hip::DeviceGuard guard(hip_stream.device_id());
  size_t ws_bytes = 0;
  HK_CALL(hk_reduce_workspace_bytes(int(in_arr->dtype()), int(nd), in_arr->shape().data(), in_arr->stride().data(),
                                    int(num_ax), axes, &ws_bytes));
  NDArray ws = Scratch(ws_bytes, in_arr->device(), stream);
  RowOutput out(out_arr, -1, stream);   // the kept elements in row-major order, laid over the output's strides
  HK_CALL(hk_reduce(int(in_arr->dtype()), int(out_arr->dtype()), in_arr->raw_data_ptr(), out.ptr(),
                    int(nd), in_arr->shape().data(), in_arr->stride().data(), int(num_ax), axes, op,
                    MutPtrOrNull(ws), ws_bytes, hip_stream));
  NDArray::MarkUsedBy({in_arr, out.array(), ws}, stream);
  out.Commit();
}
} // namespace

void ReduceSumCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_SUM, stream);
}

void ReduceMeanCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                    const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MEAN, stream);
}

void ReduceMaxCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MAX, stream);
}

void ReduceMinCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_MIN, stream);
}

void ReduceProdCuda(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                    const Stream& stream) {
  LaunchReduce(in_arr, out_arr, axes, num_ax, HK_REDUCE_PROD, stream);
}

void ReduceCuda(const NDArray& input, NDArray& output, const HTAxes& axes, ReductionType red_type,
                const Stream& stream) {
  HT_ASSERT_CUDA_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HTAxes parsed_axes = NDArrayMeta::ParseAxes(axes, int64_t(input->ndim()));
  switch (red_type) {
    case kSUM: ReduceSumCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMEAN: ReduceMeanCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMAX: ReduceMaxCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMIN: ReduceMinCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kPROD: ReduceProdCuda(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kNONE: HT_NOT_IMPLEMENTED << "Reduction type cannot be none"; break;
    default: HT_VALUE_ERROR << "Unknown reduction type: " << static_cast<int32_t>(red_type);
  }
}

// ---------------------------------------------------------------------------------------------------------
// Host twins (hetu/impl/kernel/Reduce.cc:11-73 of the reference, a oneDNN reduction there; it knows sum and
// mean only, the other three are added here).  The input may have any strides.  Two layouts get their own loop
// because they are the ones the models produce: the reduced axes are the trailing dense ones (a blocked sum per
// output), or the kept axes are the trailing dense ones (bands of columns accumulated over the reduced extent);
// anything else walks the reduced extent once per output element.  Arithmetic is fp32 for fp32 / bf16 / fp16,
// fp64 for fp64, int64 for the integer types; the mean multiplies the sum by float(1 / count) as the accelerator
// kernel does (ReduceMean.cu:9-33).
// ---------------------------------------------------------------------------------------------------------
namespace {
template <typename A> struct HostRed {
  static A identity(int op) {
    if (op == HK_REDUCE_MAX) return std::is_floating_point<A>::value ? -std::numeric_limits<A>::infinity()
                                                                    : std::numeric_limits<A>::lowest();
    if (op == HK_REDUCE_MIN) return std::is_floating_point<A>::value ? std::numeric_limits<A>::infinity()
                                                                    : std::numeric_limits<A>::max();
    return op == HK_REDUCE_PROD ? A(1) : A(0);
  }
  static A apply(int op, A a, A b) {
    switch (op) {
      case HK_REDUCE_MAX: return (a != a || a > b) ? a : b;   // a NaN wins (ReduceMax.cu:10-14)
      case HK_REDUCE_MIN: return (a != a || a < b) ? a : b;
      case HK_REDUCE_PROD: return a * b;
      default: return a + b;
    }
  }
  static A finish(int op, A v, float factor) {
    if (op != HK_REDUCE_MEAN) return v;
    if (std::is_floating_point<A>::value) return v * A(factor);
    return A(float(v) * factor);
  }
};

template <typename T> struct HostArith { using type = typename cpu::Arith<T>::type; };
template <> struct HostArith<uint8_t> { using type = int64_t; };
template <> struct HostArith<int8_t> { using type = int64_t; };
template <> struct HostArith<int16_t> { using type = int64_t; };
template <> struct HostArith<int32_t> { using type = int64_t; };
template <> struct HostArith<int64_t> { using type = int64_t; };

template <typename T, typename A> inline A host_ld(const T* p) {
  if constexpr (std::is_integral<T>::value) return A(*p);
  else return cpu::ld<T, A>(p);
}
template <typename T, typename A> inline void host_st(T* p, A v) {
  if constexpr (std::is_integral<T>::value) *p = T(v);
  else cpu::st<T, A>(p, v);
}

template <typename T, typename O>
void HostReduce(const NDArray& in, const NDArray& out, const std::vector<bool>& reduced, int op) {
  using A = typename HostArith<T>::type;
  const int64_t nd = int64_t(in->ndim());
  // kept and reduced extents with their input strides, outermost first
  std::vector<int64_t> ks, kst, rs, rst;
  for (int64_t d = 0; d < nd; ++d) {
    if (in->shape(d) == 1) continue;
    (reduced[d] ? rs : ks).push_back(in->shape(d));
    (reduced[d] ? rst : kst).push_back(in->stride(d));
  }
  int64_t n_out = 1, n_red = 1;
  for (int64_t d = 0; d < nd; ++d) (reduced[d] ? n_red : n_out) *= in->shape(d);
  const float factor = n_red > 0 ? 1.0f / float(n_red) : 0.f;
  const T* ip = in->data_ptr<T>();
  O* op_ = out->data_ptr<O>();
  auto dense_tail = [](const std::vector<int64_t>& sh, const std::vector<int64_t>& st) {
    int64_t expect = 1;
    for (int64_t i = int64_t(sh.size()) - 1; i >= 0; --i) {
      if (st[i] != expect) return false;
      expect *= sh[i];
    }
    return true;
  };
  auto offset_of = [](int64_t idx, const std::vector<int64_t>& sh, const std::vector<int64_t>& st) {
    int64_t off = 0;
    for (int64_t i = int64_t(sh.size()) - 1; i >= 0; --i) {
      off += (idx % sh[i]) * st[i];
      idx /= sh[i];
    }
    return off;
  };
  if (n_red == 0) {   // empty reduction: the identity (0 for sum / mean ... as the accelerator kernels give)
    for (int64_t o = 0; o < n_out; ++o) host_st<O, A>(op_ + o, HostRed<A>::finish(op, HostRed<A>::identity(op), factor));
    return;
  }
  const bool sum_like = op == HK_REDUCE_SUM || op == HK_REDUCE_MEAN;
  if (dense_tail(rs, rst)) {
    // rows of n_red dense elements
    cpu::parallel_rows(n_out, n_red, [&](int64_t o) {
      const T* row = ip + offset_of(o, ks, kst);
      A v;
      if (sum_like && std::is_floating_point<A>::value) {
        v = cpu::blocked_sum<A>(n_red, [&](int64_t i) { return host_ld<T, A>(row + i); });
      } else {
        v = HostRed<A>::identity(op);
        for (int64_t i = 0; i < n_red; ++i) v = HostRed<A>::apply(op, v, host_ld<T, A>(row + i));
      }
      host_st<O, A>(op_ + o, HostRed<A>::finish(op, v, factor));
    });
    return;
  }
  if (!ks.empty() && kst.back() == 1) {
    // the innermost kept axis is dense: bands of its columns accumulate over the reduced extent
    const int64_t C = ks.back(), outer = n_out / C;
    std::vector<int64_t> oks(ks.begin(), ks.end() - 1), okst(kst.begin(), kst.end() - 1);
    constexpr int64_t kBand = 64;
    const int64_t bands = (C + kBand - 1) / kBand;
    cpu::parallel_rows(outer * bands, n_red * kBand, [&](int64_t job) {
      const int64_t ob = job / bands, band = job - ob * bands;
      const int64_t c0 = band * kBand, c1 = std::min(C, c0 + kBand);
      const T* base = ip + offset_of(ob, oks, okst);
      A acc[kBand];
      for (int64_t c = 0; c < kBand; ++c) acc[c] = HostRed<A>::identity(op);
      for (int64_t r = 0; r < n_red; ++r) {
        const T* row = base + offset_of(r, rs, rst);
        if (sum_like) cpu::for_range(c0, c1, [&](int64_t c) { acc[c - c0] += host_ld<T, A>(row + c); });
        else for (int64_t c = c0; c < c1; ++c) acc[c - c0] = HostRed<A>::apply(op, acc[c - c0], host_ld<T, A>(row + c));
      }
      for (int64_t c = c0; c < c1; ++c) host_st<O, A>(op_ + ob * C + c, HostRed<A>::finish(op, acc[c - c0], factor));
    });
    return;
  }
  cpu::parallel_rows(n_out, n_red, [&](int64_t o) {
    const T* base = ip + offset_of(o, ks, kst);
    A v = HostRed<A>::identity(op);
    for (int64_t r = 0; r < n_red; ++r) v = HostRed<A>::apply(op, v, host_ld<T, A>(base + offset_of(r, rs, rst)));
    host_st<O, A>(op_ + o, HostRed<A>::finish(op, v, factor));
  });
}

void HostReduceEntry(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax, int op,
                     const char* who, const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(in_arr);
  HT_ASSERT_SAME_DEVICE(in_arr, out_arr);
  HT_ASSERT_CONTIGUOUS(out_arr);
  const int64_t nd = int64_t(in_arr->ndim());
  size_t kept = 1;
  std::vector<bool> reduced(nd, false);
  for (int64_t i = 0; i < num_ax; ++i) {
    HT_VALUE_ERROR_IF(axes[i] < 0 || axes[i] >= nd) << "axis " << axes[i] << " out of range for " << in_arr->shape();
    reduced[axes[i]] = true;
  }
  for (int64_t i = 0; i < nd; ++i)
    if (!reduced[i]) kept *= size_t(in_arr->shape(i));
  HT_ASSERT(out_arr->numel() == kept) << "output " << out_arr->shape() << " does not hold the " << kept
                                      << " kept elements of " << in_arr->shape();
  if (kept == 0) return;
  const bool widened = out_arr->dtype() == kFloat32 && in_arr->dtype() != kFloat32 &&
                       (in_arr->dtype() == kBFloat16 || in_arr->dtype() == kFloat16);
  HT_ASSERT(widened || out_arr->dtype() == in_arr->dtype())
    << who << ": the output is of the input's type, or float32 for a 16-bit floating-point input";
  HT_NOT_IMPLEMENTED_IF(widened && (op == HK_REDUCE_MAX || op == HK_REDUCE_MIN)) << who << ": max / min have no widened output";
  HT_DISPATCH_INTEGER_AND_FLOATING_TYPES(in_arr->dtype(), spec_t, who, [&]() {
    cpu::on_stream(stream, who, [=]() {   // the axis flags travel with the task; the caller's axis list is not kept
      if (widened) {
        if constexpr (std::is_same<spec_t, bfloat16>::value || std::is_same<spec_t, float16>::value)
          HostReduce<spec_t, float>(in_arr, out_arr, reduced, op);
      } else {
        HostReduce<spec_t, spec_t>(in_arr, out_arr, reduced, op);
      }
    });
  });
}
} // namespace

void ReduceSumCpu(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                  const Stream& stream) {
  HostReduceEntry(in_arr, out_arr, axes, num_ax, HK_REDUCE_SUM, "ReduceSumCpu", stream);
}
void ReduceMeanCpu(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  HostReduceEntry(in_arr, out_arr, axes, num_ax, HK_REDUCE_MEAN, "ReduceMeanCpu", stream);
}
void ReduceMaxCpu(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                  const Stream& stream) {
  HostReduceEntry(in_arr, out_arr, axes, num_ax, HK_REDUCE_MAX, "ReduceMaxCpu", stream);
}
void ReduceMinCpu(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                  const Stream& stream) {
  HostReduceEntry(in_arr, out_arr, axes, num_ax, HK_REDUCE_MIN, "ReduceMinCpu", stream);
}
void ReduceProdCpu(const NDArray& in_arr, NDArray& out_arr, const int64_t* axes, int64_t num_ax,
                   const Stream& stream) {
  HostReduceEntry(in_arr, out_arr, axes, num_ax, HK_REDUCE_PROD, "ReduceProdCpu", stream);
}

void ReduceCpu(const NDArray& input, NDArray& output, const HTAxes& axes, ReductionType red_type,
               const Stream& stream) {
  HT_ASSERT_CPU_DEVICE(input);
  HT_ASSERT_SAME_DEVICE(input, output);
  HTAxes parsed_axes = NDArrayMeta::ParseAxes(axes, int64_t(input->ndim()));
  switch (red_type) {
    case kSUM: ReduceSumCpu(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMEAN: ReduceMeanCpu(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMAX: ReduceMaxCpu(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kMIN: ReduceMinCpu(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kPROD: ReduceProdCpu(input, output, parsed_axes.data(), int64_t(parsed_axes.size()), stream); break;
    case kNONE: HT_NOT_IMPLEMENTED << "Reduction type cannot be none"; break;
    default: HT_VALUE_ERROR << "Unknown reduction type: " << static_cast<int32_t>(red_type);
  }
}

} // namespace impl
} // namespace hetu
