// Building blocks of the host ("Cpu") twins of the row-wise kernels: typed element access with the arithmetic
// type that goes with a storage type, blocked sums that the compiler can vectorise, and the row-parallel loop.
//
// The reference's host kernels are oneDNN primitives plus plain loops (hetu/impl/kernel/LayerNorm.cc:34-142,
// Softmax.cc:11-97, SoftmaxCrossEntropySparse.cc:11-126, Reduce.cc:11-73); these twins keep their pass structure
// (mean, then variance, then the output; max, then the sum of exponentials, then the output) as plain loops in the
// arithmetic type, fp32 for fp32 / bf16 / fp16 data and fp64 for fp64 data, parallel over rows with OpenMP.
#pragma once

#include "hetu/core/dtype.h"
#include "hetu/core/ndarray.h"

#include <cmath>
#include <cstdint>
#include <limits>
#include <type_traits>

namespace hetu {
namespace impl {
namespace cpu {

// arithmetic type of a storage type
template <typename T> struct Arith { using type = float; };
template <> struct Arith<double> { using type = double; };

template <typename T, typename A = typename Arith<T>::type>
inline A ld(const T* p) { return A(float(*p)); }
template <> inline double ld<double, double>(const double* p) { return *p; }
template <> inline float ld<float, float>(const float* p) { return *p; }

template <typename T, typename A>
inline void st(T* p, A v) { *p = T(float(v)); }
template <> inline void st<double, double>(double* p, double v) { *p = v; }
template <> inline void st<float, float>(float* p, float v) { *p = v; }

// Sum of f(i), i in [0, n), in kLanes independent running sums that are combined pairwise at the end: the loop
// vectorises, and the rounding error grows with n / kLanes instead of n.
constexpr int kLanes = 16;
template <typename A, typename F>
inline A blocked_sum(int64_t n, F f) {
  A acc[kLanes];
  for (int k = 0; k < kLanes; ++k) acc[k] = A(0);
  int64_t i = 0;
  for (; i + kLanes <= n; i += kLanes)
    for (int k = 0; k < kLanes; ++k) acc[k] += f(i + k);
  for (int k = 0; i < n; ++i, ++k) acc[k] += f(i);
  for (int w = kLanes / 2; w > 0; w >>= 1)
    for (int k = 0; k < w; ++k) acc[k] += acc[k + w];
  return acc[0];
}

template <typename A, typename F>
inline A blocked_max(int64_t n, F f) {
  A m = -std::numeric_limits<A>::infinity();
  bool nan = false;
  for (int64_t i = 0; i < n; ++i) {
    const A v = f(i);
    nan |= v != v;
    m = v > m ? v : m;
  }
  return nan ? std::numeric_limits<A>::quiet_NaN() : m;
}

// rows are independent in every kernel here
template <typename F>
inline void parallel_rows(int64_t rows, int64_t work_per_row, F f) {
  const bool par = rows > 1 && rows * work_per_row >= (int64_t(1) << 16);
#pragma omp parallel for schedule(static) if (par)
  for (int64_t r = 0; r < rows; ++r) f(r);
}

} // namespace cpu
} // namespace impl
} // namespace hetu
