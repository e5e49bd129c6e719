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
#include "hetu/impl/stream/CPUStream.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <type_traits>
#include <utility>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace hetu {
namespace impl {
namespace cpu {

// The computing part of a host kernel goes onto its stream: it runs after whatever the stream was given before and
// the call returns at once (stream index 0: in the calling thread, before the call returns), as the reference's
// host kernels do with CPUStream::EnqueueTask (hetu/impl/kernel/Softmax.cc:31-45 of the reference).  The task owns
// copies of the array handles it works on.  Argument checks stay in front of it, in the calling thread.
template <typename F>
inline void on_stream(const Stream& stream, const char* name, F&& body) {
  CPUStream(stream).EnqueueTask(std::function<void()>(std::forward<F>(body)), name);
}

// size of the OpenMP team of a host kernel: what SetHostKernelThreads asked for, else the runtime's default for
// the thread the kernel runs on
inline int team_size() {
  const int asked = HostKernelThreads();
#ifdef _OPENMP
  return asked > 0 ? asked : omp_get_max_threads();
#else
  return asked > 0 ? asked : 1;
#endif
}

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

// The inner loops of the host kernels exist three times: for the baseline x86-64 instruction set, for AVX2 + FMA
// and for AVX-512, picked once per process from what the processor reports (HETU_HOST_ISA=0 / 1 / 2 caps the
// choice, for tests).  A loop is written once, as a body that is inlined into three thin functions, each compiled
// for its instruction set; the callable it applies (a lambda of the calling kernel) is inlined with it.
inline int detect_isa_level() {
  int level = 0;
#if defined(__x86_64__)
  __builtin_cpu_init();
  if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c")) level = 1;
  if (level == 1 && __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
      __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512dq"))
    level = 2;
#endif
  if (const char* cap = std::getenv("HETU_HOST_ISA")) {
    const int c = std::atoi(cap);
    if (c >= 0 && c < level) level = c;
  }
  return level;
}
inline int isa_level() {
  static const int level = detect_isa_level();
  return level;
}
#if defined(__x86_64__)
#define HT_HOST_ISA_V3 __attribute__((target("avx2,fma,f16c")))
#define HT_HOST_ISA_V4 __attribute__((target("avx512f,avx512bw,avx512vl,avx512dq,avx2,fma,f16c")))
#else
#define HT_HOST_ISA_V3
#define HT_HOST_ISA_V4
#endif
#define HT_HOST_LOOP_BODY __attribute__((always_inline)) inline

// Defines NAME(args) as the choice between three compilations of BODY(args).
#define HT_HOST_ISA_VARIANTS(RET, NAME, BODY, PARAMS, ARGS)                                  \
  template <typename A, typename F> HT_HOST_ISA_V3 RET NAME##_v3 PARAMS { return BODY<A> ARGS; } \
  template <typename A, typename F> HT_HOST_ISA_V4 RET NAME##_v4 PARAMS { return BODY<A> ARGS; } \
  template <typename A, typename F> inline RET NAME PARAMS {                                 \
    switch (isa_level()) {                                                                   \
      case 2: return NAME##_v4<A> ARGS;                                                      \
      case 1: return NAME##_v3<A> ARGS;                                                      \
      default: return BODY<A> ARGS;                                                          \
    }                                                                                        \
  }

// Sum of f(i), i in [0, n), in kLanes independent running sums that are combined pairwise at the end: the loop
// vectorises, and the rounding error grows with n / kLanes instead of n.
constexpr int kLanes = 16;
template <typename A, typename F>
HT_HOST_LOOP_BODY A blocked_sum_body(int64_t n, F& f) {
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
HT_HOST_ISA_VARIANTS(A, blocked_sum, blocked_sum_body, (int64_t n, F f), (n, f))

// Maximum of f(i), i in [0, n), NaN if any term is: kLanes running maxima and NaN flags side by side (selects
// between lanes, which vectorise where a single running maximum would not), combined at the end.
template <typename A, typename F>
HT_HOST_LOOP_BODY A blocked_max_body(int64_t n, F& f) {
  A mx[kLanes];
  int bad[kLanes];
  for (int k = 0; k < kLanes; ++k) { mx[k] = -std::numeric_limits<A>::infinity(); bad[k] = 0; }
  int64_t i = 0;
  for (; i + kLanes <= n; i += kLanes) {
    A v[kLanes];
    for (int k = 0; k < kLanes; ++k) v[k] = f(i + k);
    for (int k = 0; k < kLanes; ++k) {
      bad[k] |= v[k] != v[k] ? 1 : 0;
      mx[k] = v[k] > mx[k] ? v[k] : mx[k];
    }
  }
  for (int k = 0; i < n; ++i, ++k) {
    const A v = f(i);
    bad[k] |= v != v ? 1 : 0;
    mx[k] = v > mx[k] ? v : mx[k];
  }
  A m = mx[0];
  int nan = bad[0];
  for (int k = 1; k < kLanes; ++k) { m = mx[k] > m ? mx[k] : m; nan |= bad[k]; }
  return nan ? std::numeric_limits<A>::quiet_NaN() : m;
}
HT_HOST_ISA_VARIANTS(A, blocked_max, blocked_max_body, (int64_t n, F f), (n, f))

// f(i) for i in [begin, end), in order, in the calling thread: the element-wise loop of a kernel's row
template <typename A, typename F>
HT_HOST_LOOP_BODY void for_range_body(int64_t begin, int64_t end, F& f) {
  for (int64_t i = begin; i < end; ++i) f(i);
}
HT_HOST_ISA_VARIANTS(void, for_range_any, for_range_body, (int64_t begin, int64_t end, F f), (begin, end, f))
template <typename F>
inline void for_range(int64_t begin, int64_t end, F f) { for_range_any<void>(begin, end, f); }

// A loop body written once for a run-time element step and compiled a second time for step 1, the case whose
// loads and stores are contiguous and vectorise: f receives a callable that returns the step.
struct UnitStep { constexpr int64_t operator()() const { return 1; } };
struct AnyStep { int64_t value; int64_t operator()() const { return value; } };
template <typename F>
inline void with_step(int64_t step, F f) {
  if (step == 1) f(UnitStep{});
  else f(AnyStep{step});
}

// exp for the float arithmetic of the host kernels, written without a branch or a library call so that the loops
// around it vectorise: x = n ln2 + r with |r| <= ln2 / 2 (n rounded by the 1.5 * 2^23 trick, ln2 split in two so
// that n * ln2_hi is exact), a degree-6 polynomial in r, and 2^n applied through the exponent bits in two factors,
// which keeps gradual underflow.  Within 2 units in the last place of the exact value; exp(-inf) = 0, overflow
// gives +inf, NaN stays NaN.  float64 data keeps std::exp.
inline float exp_(float x) {
  const float lo = -104.f, hi = 89.f;
  const float xc = x < lo ? lo : (x > hi ? hi : x);          // NaN passes through
  const float xs = xc == xc ? xc : 0.f;                      // the exponent is taken from a number
  const float magic = 12582912.f;                            // 1.5 * 2^23
  const float nf = (xs * 1.44269504088896341f + magic) - magic;
  float r = xc - nf * 0.693359375f;                          // ln2_hi: 10 significant bits
  r = r - nf * -2.12194440e-4f;                              // ln2_lo
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  p = p * (r * r) + r + 1.f;
  const int32_t n = int32_t(nf);
  const int32_t n1 = n >> 1, n2 = n - n1;                    // both within [-75, 65]
  const uint32_t b1 = uint32_t(n1 + 127) << 23, b2 = uint32_t(n2 + 127) << 23;
  float s1, s2;
  std::memcpy(&s1, &b1, 4);
  std::memcpy(&s2, &b2, 4);
  return p * s1 * s2;
}
inline double exp_(double x) { return std::exp(x); }

// x op y on one element of storage type T, op being 0 add, 1 subtract, 2 multiply, 3 divide (the values of the
// HK_BINARY_* constants).  Floating-point types compute in their arithmetic type and round once; integers wrap in
// their own width, and a division by zero gives 0 instead of a trap.
template <typename T>
inline T binary_op(int op, T x, T y) {
  if constexpr (std::is_integral<T>::value) {
    using U = typename std::make_unsigned<T>::type;
    switch (op) {
      case 0: return T(U(U(x) + U(y)));
      case 1: return T(U(U(x) - U(y)));
      case 2: return T(U(U(x) * U(y)));
      default:
        if (y == T(0)) return T(0);
        if constexpr (std::is_signed<T>::value) {
          if (y == T(-1)) return T(U(U(0) - U(x)));   // the one quotient that does not fit
        }
        return T(x / y);
    }
  } else {
    using A = typename Arith<T>::type;
    const A a = ld<T, A>(&x), b = ld<T, A>(&y);
    const A r = op == 0 ? a + b : op == 1 ? a - b : op == 2 ? a * b : a / b;
    T out;
    st<T, A>(&out, r);
    return out;
  }
}

// the negation of one element; integers wrap
template <typename T>
inline T negate(T x) {
  if constexpr (std::is_integral<T>::value) {
    using U = typename std::make_unsigned<T>::type;
    return T(U(U(0) - U(x)));
  } else {
    using A = typename Arith<T>::type;
    T out;
    st<T, A>(&out, -ld<T, A>(&x));
    return out;
  }
}

// f(i) for i in [0, n), shared out over the OpenMP team when there is enough of it
template <typename F>
inline void parallel_for(int64_t n, F f) {
  // pieces of 8192 elements, each a plain loop in the instruction set of the processor
  constexpr int64_t kPiece = 8192;
  const int64_t pieces = (n + kPiece - 1) / kPiece;
#pragma omp parallel for schedule(static) num_threads(team_size()) if (n >= (int64_t(1) << 16))
  for (int64_t p = 0; p < pieces; ++p) for_range(p * kPiece, std::min(n, (p + 1) * kPiece), f);
}

// Walks a dense row-major array of `nd` dimensions run by run along the last dimension: f(out_offset, a_offset,
// b_offset) is called once per run with the element offsets of its first element in the output and in two operands
// laid out by the strides sa / sb (0 where an operand repeats); the run has shape[nd - 1] elements, sa[nd - 1] /
// sb[nd - 1] apart in the operands.  Runs are shared out over the OpenMP team.
template <typename F>
inline void for_each_run(int nd, const int64_t* shape, const int64_t* sa, const int64_t* sb, F f) {
  if (nd == 0) { f(int64_t(0), int64_t(0), int64_t(0)); return; }
  const int64_t inner = shape[nd - 1];
  int64_t runs = 1;
  for (int d = 0; d < nd - 1; ++d) runs *= shape[d];
  const bool par = runs > 1 && runs * inner >= (int64_t(1) << 16);
#pragma omp parallel for schedule(static) num_threads(team_size()) if (par)
  for (int64_t r = 0; r < runs; ++r) {
    int64_t rem = r, oa = 0, ob = 0;
    for (int d = nd - 2; d >= 0; --d) {
      const int64_t q = rem / shape[d], c = rem - q * shape[d];
      oa += c * sa[d];
      ob += c * sb[d];
      rem = q;
    }
    f(r * inner, oa, ob);
  }
}

// rows are independent in every kernel here
template <typename F>
inline void parallel_rows(int64_t rows, int64_t work_per_row, F f) {
  const bool par = rows > 1 && rows * work_per_row >= (int64_t(1) << 16);
#pragma omp parallel for schedule(static) num_threads(team_size()) if (par)
  for (int64_t r = 0; r < rows; ++r) f(r);
}

} // namespace cpu
} // namespace impl
} // namespace hetu
