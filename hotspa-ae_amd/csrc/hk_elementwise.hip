// Element-wise kernels: exp / log / negate / sqrt, array-with-constant and
// array-with-array add / sub / mul / div with broadcasting.  One 16-byte
// vector per thread and a grid that covers the array once (the shape that
// streams fastest on this part); operands that broadcast along rows or
// columns are read as one value or one cached vector.  Arithmetic is fp32 for
// the 16-bit types (one rounding at the store), fp64 for fp64.  Outputs may
// alias an input of the same shape (every thread reads its elements before it
// writes them).
#include "hk_common.h"

#include <type_traits>

namespace hk {

enum { EW_ADD = 0, EW_SUB = 1, EW_MUL = 2, EW_DIV = 3 };
enum { EW_EXP = 0, EW_LOG = 1, EW_NEG = 2, EW_SQRT = 3 };

template <int OP, typename CT>
__device__ __forceinline__ CT ew_bin(CT a, CT b) {
  if constexpr (OP == EW_ADD) return a + b;
  else if constexpr (OP == EW_SUB) return a - b;
  else if constexpr (OP == EW_MUL) return a * b;
  else return a / b;
}

template <int OP, typename CT>
__device__ __forceinline__ CT ew_un(CT a) {
  if constexpr (OP == EW_EXP) {
    if constexpr (std::is_same<CT, double>::value) return exp(a); else return expf(a);
  } else if constexpr (OP == EW_LOG) {
    if constexpr (std::is_same<CT, double>::value) return log(a); else return logf(a);
  } else if constexpr (OP == EW_NEG) {
    return -a;
  } else {
    if constexpr (std::is_same<CT, double>::value) return sqrt(a); else return sqrtf(a);
  }
}

// arithmetic type: fp32 for the 16-bit floats, the type itself for fp64 and the integers (which wrap as the
// type does: the result of the promoted operation is converted back on the store)
template <typename T> struct EwCT { using type = typename std::conditional<std::is_integral<T>::value, T, float>::type; };
template <> struct EwCT<double> { using type = double; };

template <typename T>
__device__ __forceinline__ typename EwCT<T>::type ew_load(const T* p) {
  if constexpr (std::is_integral<T>::value) return *p;
  else return typename EwCT<T>::type(Cvt<T>::load(p));
}
template <typename T>
__device__ __forceinline__ void ew_store(T* p, typename EwCT<T>::type v) {
  if constexpr (std::is_integral<T>::value) *p = v;
  else Cvt<T>::store(p, v);
}
template <typename T> constexpr bool ew_vectorised() {
  return !std::is_same<T, double>::value && !std::is_integral<T>::value;
}

// ---------------------------------------------------------------------------
// unary, and binary with a constant (REV: constant op x instead of x op constant)
// ---------------------------------------------------------------------------
template <typename T, int OP>
__global__ __launch_bounds__(kStreamThreads) void ew_unary_vec_kernel(const T* in, T* out, int64_t nvec) {
  constexpr int VEC = VecIO<T>::N;
  const int64_t v = int64_t(blockIdx.x) * kStreamThreads + threadIdx.x;
  if (v >= nvec) return;
  float f[VEC];
  VecIO<T>::unpack(ld16(in + v * VEC), f);
#pragma unroll
  for (int j = 0; j < VEC; ++j) f[j] = ew_un<OP, float>(f[j]);
  st16_stream(out + v * VEC, VecIO<T>::pack(f));
}

template <typename T, int OP>
__global__ __launch_bounds__(256) void ew_unary_scalar_kernel(const T* in, T* out, int64_t n) {
  using CT = typename EwCT<T>::type;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) ew_store(out + i, CT(ew_un<OP, CT>(ew_load(in + i))));
}

template <typename T, int OP, bool REV>
__global__ __launch_bounds__(kStreamThreads) void ew_const_vec_kernel(const T* in, float c, T* out,
                                                                      int64_t nvec) {
  constexpr int VEC = VecIO<T>::N;
  const int64_t v = int64_t(blockIdx.x) * kStreamThreads + threadIdx.x;
  if (v >= nvec) return;
  float f[VEC];
  VecIO<T>::unpack(ld16(in + v * VEC), f);
#pragma unroll
  for (int j = 0; j < VEC; ++j) f[j] = REV ? ew_bin<OP, float>(c, f[j]) : ew_bin<OP, float>(f[j], c);
  st16_stream(out + v * VEC, VecIO<T>::pack(f));
}

template <typename T, int OP, bool REV>
__global__ __launch_bounds__(256) void ew_const_scalar_kernel(const T* in, double c, T* out,
                                                              int64_t n) {
  using CT = typename EwCT<T>::type;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  const CT x = ew_load(in + i), k = CT(c);
  ew_store(out + i, CT(REV ? ew_bin<OP, CT>(k, x) : ew_bin<OP, CT>(x, k)));
}

// ---------------------------------------------------------------------------
// binary with broadcasting
// ---------------------------------------------------------------------------
// How an operand maps onto the [rows, cols] output of the two-dimensional kernel.
enum { EW_FULL = 0, EW_PER_ROW = 1, EW_PER_COL = 2, EW_SINGLE = 3 };

// An operand's 16 bytes (or its single value) as loaded, before any unpacking: both operands' loads are issued
// back to back and waited for once.
template <typename T, int MODE>
struct EwRaw {
  u32x4 vec;
  float one;
  __device__ __forceinline__ void load(const T* p, int64_t v, int64_t r, int64_t c) {
    constexpr int VEC = VecIO<T>::N;
    if constexpr (MODE == EW_FULL) vec = ld16(p + v * VEC);
    else if constexpr (MODE == EW_PER_COL) vec = ld16_keep(p + c * VEC);
    else if constexpr (MODE == EW_PER_ROW) one = Cvt<T>::load(p + r);
    else one = Cvt<T>::load(p);
  }
  __device__ __forceinline__ void unpack(float* f) const {
    constexpr int VEC = VecIO<T>::N;
    if constexpr (MODE == EW_FULL || MODE == EW_PER_COL) {
      VecIO<T>::unpack(vec, f);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) f[j] = one;
    }
  }
};

// out[r, c] = a[..] op b[..] over a [rows, cols] output; cols_vec = vectors per output row; AM / BM say how
// each operand maps onto the output.
template <typename T, int OP, int AM, int BM>
__global__ __launch_bounds__(kStreamThreads) void ew_binary_2d_vec_kernel(const T* a, const T* b, T* out, uint32_t nvec,
                                                               uint32_t cols_vec) {
  constexpr int VEC = VecIO<T>::N;
  const uint32_t v = blockIdx.x * uint32_t(kStreamThreads) + threadIdx.x;
  if (v >= nvec) return;
  uint32_t r = 0, c = v;
  if constexpr (AM != EW_FULL || BM != EW_FULL) {
    r = v / cols_vec;
    c = v - r * cols_vec;
  }
  EwRaw<T, AM> ra;
  EwRaw<T, BM> rb;
  ra.load(a, v, r, c);
  rb.load(b, v, r, c);
  float fa[VEC], fb[VEC];
  ra.unpack(fa);
  rb.unpack(fb);
#pragma unroll
  for (int j = 0; j < VEC; ++j) fa[j] = ew_bin<OP, float>(fa[j], fb[j]);
  st16_stream(out + size_t(v) * VEC, VecIO<T>::pack(fa));
}

struct EwDims {
  int ndim;
  int64_t shape[8];
  int64_t astride[8];
  int64_t bstride[8];
};

// any shape, any strides, one element per thread
template <typename T, int OP>
__global__ __launch_bounds__(256) void ew_binary_generic_kernel(const T* a, const T* b,
                                                                T* out, EwDims d, int64_t n) {
  using CT = typename EwCT<T>::type;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  int64_t rem = i, oa = 0, ob = 0;
  for (int k = d.ndim - 1; k >= 0; --k) {
    const int64_t q = rem / d.shape[k];
    const int64_t idx = rem - q * d.shape[k];
    rem = q;
    oa += idx * d.astride[k];
    ob += idx * d.bstride[k];
  }
  ew_store(out + i, CT(ew_bin<OP, CT>(ew_load(a + oa), ew_load(b + ob))));
}

// out = broadcast(a) [* c]: a dense output filled from an operand that maps onto it in one of the four modes.
// What a reduction's backward does with the gradient of its output.
template <typename T, int AM, bool MUL>
__global__ __launch_bounds__(256) void ew_broadcast_2d_vec_kernel(const T* a, float c, T* out, uint32_t nvec,
                                                                  uint32_t cols_vec) {
  constexpr int VEC = VecIO<T>::N;
  const uint32_t v = blockIdx.x * 256u + threadIdx.x;
  if (v >= nvec) return;
  uint32_t r = 0, col = v;
  if constexpr (AM != EW_FULL) {
    r = v / cols_vec;
    col = v - r * cols_vec;
  }
  EwRaw<T, AM> ra;
  ra.load(a, v, r, col);
  float f[VEC];
  ra.unpack(f);
  if constexpr (MUL) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] *= c;
  }
  st16_stream(out + size_t(v) * VEC, VecIO<T>::pack(f));
}

template <typename T, bool MUL>
__global__ __launch_bounds__(256) void ew_broadcast_generic_kernel(const T* a, double c, T* out, EwDims d,
                                                                   int64_t n) {
  using CT = typename EwCT<T>::type;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  int64_t rem = i, oa = 0;
  for (int k = d.ndim - 1; k >= 0; --k) {
    const int64_t q = rem / d.shape[k];
    oa += (rem - q * d.shape[k]) * d.astride[k];
    rem = q;
  }
  const CT x = ew_load(a + oa);
  ew_store(out + i, MUL ? CT(x * CT(c)) : x);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static inline unsigned blocks_for(int64_t n) { return unsigned((n + 255) / 256); }
static inline unsigned stream_blocks_for(int64_t nvec) { return unsigned((nvec + kStreamThreads - 1) / kStreamThreads); }

template <typename T, int OP>
static int unary_launch(const void* in, void* out, int64_t n, hipStream_t s) {
  HK_REQUIRE((n + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_unary: array too large");
  profile_before(s);
  if constexpr (ew_vectorised<T>()) {
    constexpr int VEC = VecIO<T>::N;
    if (n % VEC == 0 && aligned16(in) && aligned16(out)) {
      HK_LAUNCH((ew_unary_vec_kernel<T, OP>), dim3(stream_blocks_for(n / VEC)), dim3(kStreamThreads), 0, s,
                         static_cast<const T*>(in), static_cast<T*>(out), n / VEC);
      profile_after(s);
      return launch_check("ew_unary_vec_kernel");
    }
  }
  HK_LAUNCH((ew_unary_scalar_kernel<T, OP>), dim3(blocks_for(n)), dim3(256), 0, s,
                     static_cast<const T*>(in), static_cast<T*>(out), n);
  profile_after(s);
  return launch_check("ew_unary_scalar_kernel");
}

template <typename T, int OP, bool REV>
static int const_launch(const void* in, double c, void* out, int64_t n, hipStream_t s) {
  HK_REQUIRE((n + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_binary_const: array too large");
  c = round_const<T>(c);
  profile_before(s);
  if constexpr (ew_vectorised<T>()) {
    constexpr int VEC = VecIO<T>::N;
    if (n % VEC == 0 && aligned16(in) && aligned16(out)) {
      HK_LAUNCH((ew_const_vec_kernel<T, OP, REV>), dim3(stream_blocks_for(n / VEC)), dim3(kStreamThreads), 0, s,
                         static_cast<const T*>(in), float(c), static_cast<T*>(out), n / VEC);
      profile_after(s);
      return launch_check("ew_const_vec_kernel");
    }
  }
  HK_LAUNCH((ew_const_scalar_kernel<T, OP, REV>), dim3(blocks_for(n)), dim3(256), 0, s,
                     static_cast<const T*>(in), c, static_cast<T*>(out), n);
  profile_after(s);
  return launch_check("ew_const_scalar_kernel");
}

// Drops extent-1 dims and merges neighbours that both operands (and the dense output) walk contiguously.
static EwDims merge_dims(int ndim, const int64_t* shape, const int64_t* as, const int64_t* bs) {
  EwDims d{};
  for (int i = 0; i < ndim; ++i) {
    if (shape[i] == 1) continue;
    if (d.ndim > 0) {
      const int k = d.ndim - 1;
      if (d.astride[k] == as[i] * shape[i] && d.bstride[k] == bs[i] * shape[i]) {
        d.shape[k] *= shape[i];
        d.astride[k] = as[i];
        d.bstride[k] = bs[i];
        continue;
      }
    }
    d.shape[d.ndim] = shape[i];
    d.astride[d.ndim] = as[i];
    d.bstride[d.ndim] = bs[i];
    ++d.ndim;
  }
  if (d.ndim == 0) {   // a single element
    d.ndim = 1;
    d.shape[0] = 1; d.astride[0] = 0; d.bstride[0] = 0;
  }
  return d;
}

// mode of an operand over a [rows, cols] output from its two merged strides; -1: none of the four
static int operand_mode(int64_t rows, int64_t cols, int64_t s0, int64_t s1) {
  const bool row_fixed = rows == 1 || s0 == 0;
  const bool col_fixed = cols == 1 || s1 == 0;
  if (row_fixed && col_fixed) return EW_SINGLE;
  if (col_fixed) return (s0 == 1) ? EW_PER_ROW : -1;
  if (s1 != 1) return -1;
  // a single row walked with unit stride is the whole array (two dense arrays of one shape merge to this)
  if (rows == 1) return EW_FULL;
  if (row_fixed) return EW_PER_COL;
  return s0 == cols ? EW_FULL : -1;
}

template <typename T, int OP>
static int binary_launch(const void* a, const void* b, void* out, const EwDims& d, int64_t n, hipStream_t s) {
  HK_REQUIRE((n + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_binary: array too large");
  const T* pa = static_cast<const T*>(a);
  const T* pb = static_cast<const T*>(b);
  T* po = static_cast<T*>(out);
  profile_before(s);
  if constexpr (ew_vectorised<T>()) {
    constexpr int VEC = VecIO<T>::N;
    if (d.ndim <= 2) {
      const int64_t rows = d.ndim == 2 ? d.shape[0] : 1;
      const int64_t cols = d.ndim == 2 ? d.shape[1] : d.shape[0];
      const int64_t a0 = d.ndim == 2 ? d.astride[0] : 0, a1 = d.ndim == 2 ? d.astride[1] : d.astride[0];
      const int64_t b0 = d.ndim == 2 ? d.bstride[0] : 0, b1 = d.ndim == 2 ? d.bstride[1] : d.bstride[0];
      const int am = operand_mode(rows, cols, a0, a1), bm = operand_mode(rows, cols, b0, b1);
      auto vec_ok = [&](const void* p, int mode) {
        return mode == EW_PER_ROW || mode == EW_SINGLE || aligned16(p);
      };
      // one full operand, the other in any of the four modes; two broadcast operands take the generic kernel
      if (am >= 0 && bm >= 0 && (am == EW_FULL || bm == EW_FULL) && cols % VEC == 0 && aligned16(out) &&
          vec_ok(a, am) && vec_ok(b, bm) && n / VEC < 0x7fffffffLL) {
        const uint32_t nvec = uint32_t(n / VEC), cols_vec = uint32_t(cols / VEC);
        const dim3 grid(stream_blocks_for(nvec)), block(kStreamThreads);
#define HK_EW_2D(AM, BM) \
  HK_LAUNCH((ew_binary_2d_vec_kernel<T, OP, AM, BM>), grid, block, 0, s, pa, pb, po, nvec, cols_vec)
        if (am == EW_FULL) {
          switch (bm) {
            case EW_FULL: HK_EW_2D(EW_FULL, EW_FULL); break;
            case EW_PER_ROW: HK_EW_2D(EW_FULL, EW_PER_ROW); break;
            case EW_PER_COL: HK_EW_2D(EW_FULL, EW_PER_COL); break;
            default: HK_EW_2D(EW_FULL, EW_SINGLE); break;
          }
        } else {
          switch (am) {
            case EW_PER_ROW: HK_EW_2D(EW_PER_ROW, EW_FULL); break;
            case EW_PER_COL: HK_EW_2D(EW_PER_COL, EW_FULL); break;
            default: HK_EW_2D(EW_SINGLE, EW_FULL); break;
          }
        }
#undef HK_EW_2D
        profile_after(s);
        return launch_check("ew_binary_2d_vec_kernel");
      }
    }
  }
  HK_LAUNCH((ew_binary_generic_kernel<T, OP>), dim3(blocks_for(n)), dim3(256), 0, s, pa, pb, po, d, n);
  profile_after(s);
  return launch_check("ew_binary_generic_kernel");
}

template <typename T, bool MUL>
static int broadcast_launch(const void* a, double c, void* out, const EwDims& d, int64_t n, hipStream_t s) {
  HK_REQUIRE((n + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_broadcast: array too large");
  const T* pa = static_cast<const T*>(a);
  T* po = static_cast<T*>(out);
  c = round_const<T>(c);
  profile_before(s);
  if constexpr (ew_vectorised<T>()) {
    constexpr int VEC = VecIO<T>::N;
    if (d.ndim <= 2) {
      const int64_t rows = d.ndim == 2 ? d.shape[0] : 1;
      const int64_t cols = d.ndim == 2 ? d.shape[1] : d.shape[0];
      const int64_t a0 = d.ndim == 2 ? d.astride[0] : 0, a1 = d.ndim == 2 ? d.astride[1] : d.astride[0];
      const int am = operand_mode(rows, cols, a0, a1);
      const bool a_ok = am == EW_PER_ROW || am == EW_SINGLE || aligned16(a);
      if (am >= 0 && cols % VEC == 0 && aligned16(out) && a_ok && n / VEC < 0x7fffffffLL) {
        const uint32_t nvec = uint32_t(n / VEC), cols_vec = uint32_t(cols / VEC);
        const dim3 grid(blocks_for(nvec)), block(256);
#define HK_EW_BC(AM) \
  HK_LAUNCH((ew_broadcast_2d_vec_kernel<T, AM, MUL>), grid, block, 0, s, pa, float(c), po, nvec, cols_vec)
        switch (am) {
          case EW_FULL: HK_EW_BC(EW_FULL); break;
          case EW_PER_ROW: HK_EW_BC(EW_PER_ROW); break;
          case EW_PER_COL: HK_EW_BC(EW_PER_COL); break;
          default: HK_EW_BC(EW_SINGLE); break;
        }
#undef HK_EW_BC
        profile_after(s);
        return launch_check("ew_broadcast_2d_vec_kernel");
      }
    }
  }
  HK_LAUNCH((ew_broadcast_generic_kernel<T, MUL>), dim3(blocks_for(n)), dim3(256), 0, s, pa, c, po, d, n);
  profile_after(s);
  return launch_check("ew_broadcast_generic_kernel");
}

#define HK_EW_FLOAT_CASES(CALL)                                          \
    case HK_FLOAT32: { using T = float; return CALL; }                   \
    case HK_BFLOAT16: { using T = bf16; return CALL; }                   \
    case HK_FLOAT16: { using T = fp16; return CALL; }                    \
    case HK_FLOAT64: { using T = double; return CALL; }
#define HK_EW_INT_CASES(CALL)                                            \
    case HK_UINT8: { using T = uint8_t; return CALL; }                   \
    case HK_INT8: { using T = int8_t; return CALL; }                     \
    case HK_INT16: { using T = int16_t; return CALL; }                   \
    case HK_INT32: { using T = int32_t; return CALL; }                   \
    case HK_INT64: { using T = int64_t; return CALL; }
#define HK_EW_UNSUPPORTED(dtype, who)                                    \
    default:                                                             \
      set_last_error("%s: not implemented for dtype %d", who, dtype);    \
      return HK_ERR_UNSUPPORTED;
// floating types only (exp, log, sqrt), or the integers as well (the arithmetic, negation, broadcast)
#define HK_EW_TYPES(dtype, who, CALL) \
  switch (dtype) { HK_EW_FLOAT_CASES(CALL) HK_EW_UNSUPPORTED(dtype, who) }
#define HK_EW_ALL_TYPES(dtype, who, CALL) \
  switch (dtype) { HK_EW_FLOAT_CASES(CALL) HK_EW_INT_CASES(CALL) HK_EW_UNSUPPORTED(dtype, who) }

template <int OP>
static int unary_typed(int dtype, const void* in, void* out, int64_t n, hipStream_t s) {
  if constexpr (OP == EW_NEG) {
    HK_EW_ALL_TYPES(dtype, "hk_unary", (unary_launch<T, OP>(in, out, n, s)));
  } else {
    HK_EW_TYPES(dtype, "hk_unary", (unary_launch<T, OP>(in, out, n, s)));
  }
}
template <int OP, bool REV>
static int const_typed(int dtype, const void* in, double c, void* out, int64_t n, hipStream_t s) {
  HK_EW_ALL_TYPES(dtype, "hk_binary_const", (const_launch<T, OP, REV>(in, c, out, n, s)));
}
template <int OP>
static int binary_typed(int dtype, const void* a, const void* b, void* out, const EwDims& d, int64_t n,
                        hipStream_t s) {
  HK_EW_ALL_TYPES(dtype, "hk_binary", (binary_launch<T, OP>(a, b, out, d, n, s)));
}

template <bool MUL>
static int broadcast_typed(int dtype, const void* a, double c, void* out, const EwDims& d, int64_t n,
                           hipStream_t s) {
  HK_EW_ALL_TYPES(dtype, "hk_broadcast", (broadcast_launch<T, MUL>(a, c, out, d, n, s)));
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_unary(int op, int dtype, const void* in, void* out, int64_t numel, hkStream_t stream) {
  HK_REQUIRE(numel >= 0, HK_ERR_INVALID, "hk_unary: negative size");
  if (numel == 0) return HK_OK;
  HK_REQUIRE(in && out, HK_ERR_INVALID, "hk_unary: null input/output");
  hipStream_t s = as_hip(stream);
  switch (op) {
    case HK_UNARY_EXP: return unary_typed<EW_EXP>(dtype, in, out, numel, s);
    case HK_UNARY_LOG: return unary_typed<EW_LOG>(dtype, in, out, numel, s);
    case HK_UNARY_NEG: return unary_typed<EW_NEG>(dtype, in, out, numel, s);
    case HK_UNARY_SQRT: return unary_typed<EW_SQRT>(dtype, in, out, numel, s);
    default: set_last_error("hk_unary: unknown op %d", op); return HK_ERR_INVALID;
  }
}

int hk_binary_const(int op, int dtype, const void* in, double scalar, int scalar_first, void* out, int64_t numel,
                    hkStream_t stream) {
  HK_REQUIRE(numel >= 0, HK_ERR_INVALID, "hk_binary_const: negative size");
  if (numel == 0) return HK_OK;
  HK_REQUIRE(in && out, HK_ERR_INVALID, "hk_binary_const: null input/output");
  hipStream_t s = as_hip(stream);
  const bool rev = scalar_first != 0;
  switch (op) {
    case HK_BINARY_ADD: return const_typed<EW_ADD, false>(dtype, in, scalar, out, numel, s);
    case HK_BINARY_MUL: return const_typed<EW_MUL, false>(dtype, in, scalar, out, numel, s);
    case HK_BINARY_SUB:
      return rev ? const_typed<EW_SUB, true>(dtype, in, scalar, out, numel, s)
                 : const_typed<EW_SUB, false>(dtype, in, scalar, out, numel, s);
    case HK_BINARY_DIV:
      return rev ? const_typed<EW_DIV, true>(dtype, in, scalar, out, numel, s)
                 : const_typed<EW_DIV, false>(dtype, in, scalar, out, numel, s);
    default: set_last_error("hk_binary_const: unknown op %d", op); return HK_ERR_INVALID;
  }
}

int hk_binary(int op, int dtype, const void* a, const void* b, void* out, int ndim, const int64_t* out_shape,
              const int64_t* a_strides, const int64_t* b_strides, hkStream_t stream) {
  HK_REQUIRE(ndim >= 0 && ndim <= 8, HK_ERR_INVALID, "hk_binary: ndim %d outside [0, 8]", ndim);
  HK_REQUIRE(ndim == 0 || (out_shape && a_strides && b_strides), HK_ERR_INVALID, "hk_binary: null shape/strides");
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    HK_REQUIRE(out_shape[i] >= 0, HK_ERR_INVALID, "hk_binary: negative extent");
    HK_REQUIRE(a_strides[i] >= 0 && b_strides[i] >= 0, HK_ERR_INVALID, "hk_binary: negative stride");
    n *= out_shape[i];
  }
  if (n == 0) return HK_OK;
  HK_REQUIRE(a && b && out, HK_ERR_INVALID, "hk_binary: null input/output");
  const EwDims d = merge_dims(ndim, out_shape, a_strides, b_strides);
  hipStream_t s = as_hip(stream);
  switch (op) {
    case HK_BINARY_ADD: return binary_typed<EW_ADD>(dtype, a, b, out, d, n, s);
    case HK_BINARY_SUB: return binary_typed<EW_SUB>(dtype, a, b, out, d, n, s);
    case HK_BINARY_MUL: return binary_typed<EW_MUL>(dtype, a, b, out, d, n, s);
    case HK_BINARY_DIV: return binary_typed<EW_DIV>(dtype, a, b, out, d, n, s);
    default: set_last_error("hk_binary: unknown op %d", op); return HK_ERR_INVALID;
  }
}

int hk_broadcast(int dtype, const void* in, int multiply, double scalar, void* out, int ndim,
                 const int64_t* out_shape, const int64_t* in_strides, hkStream_t stream) {
  HK_REQUIRE(ndim >= 0 && ndim <= 8, HK_ERR_INVALID, "hk_broadcast: ndim %d outside [0, 8]", ndim);
  HK_REQUIRE(ndim == 0 || (out_shape && in_strides), HK_ERR_INVALID, "hk_broadcast: null shape/strides");
  int64_t n = 1;
  for (int i = 0; i < ndim; ++i) {
    HK_REQUIRE(out_shape[i] >= 0, HK_ERR_INVALID, "hk_broadcast: negative extent");
    HK_REQUIRE(in_strides[i] >= 0, HK_ERR_INVALID, "hk_broadcast: negative stride");
    n *= out_shape[i];
  }
  if (n == 0) return HK_OK;
  HK_REQUIRE(in && out, HK_ERR_INVALID, "hk_broadcast: null input/output");
  const EwDims d = merge_dims(ndim, out_shape, in_strides, in_strides);
  hipStream_t s = as_hip(stream);
  return multiply ? broadcast_typed<true>(dtype, in, scalar, out, d, n, s)
                  : broadcast_typed<false>(dtype, in, scalar, out, d, n, s);
}

} // extern "C"
