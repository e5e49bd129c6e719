// Local kernels of the vocabulary-parallel cross-entropy: every device holds the
// columns [vocab_start, vocab_end) of the logits; what crosses devices (the row
// maximum, the sum of exponentials, the picked logit) is reduced by the caller
// between these kernels.
#include "hk_common.h"

#include <type_traits>

namespace hk {

// One thread per row: the logit at the label when the label falls into this shard, else 0; rows whose
// label is `ignored_index` get 0 in both outputs.  lse of the other rows is left as the caller filled it.
template <typename T>
__global__ __launch_bounds__(256)
void vocab_ce_gather_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels, int64_t rows,
                            int64_t cols, int64_t vocab_start, int64_t vocab_end, int64_t ignored_index,
                            T* __restrict__ picked, T* __restrict__ lse) {
  const int64_t r = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (r >= rows) return;
  const int64_t label = labels[r];
  T zero;
  __builtin_memset(&zero, 0, sizeof(T));
  if (label == ignored_index) {
    picked[r] = zero;
    lse[r] = zero;
    return;
  }
  if (label < vocab_start || label >= vocab_end) picked[r] = zero;
  else picked[r] = logits[r * cols + (label - vocab_start)];
}

// out[r, c] = (softmax[r, c] - [c == labels[r] - vocab_start]) * grad_loss[r]; the comparison is made on
// unsigned 64-bit values, so a label outside the shard (or a negative one) matches no column.
template <typename T>
__global__ __launch_bounds__(kStreamThreads)
void vocab_ce_bwd_vec_kernel(const T* softmax, const int64_t* __restrict__ labels, const T* __restrict__ grad_loss,
                             T* out, uint32_t nvec, uint32_t cols_vec, int64_t vocab_start) {
  constexpr int VEC = VecIO<T>::N;
  const uint32_t v = blockIdx.x * uint32_t(kStreamThreads) + threadIdx.x;
  if (v >= nvec) return;
  const uint32_t r = v / cols_vec;
  const uint32_t c0 = (v - r * cols_vec) * VEC;
  const u32x4 raw = ld16(softmax + size_t(v) * VEC);
  // a wavefront almost always lies inside one row: then the row's label and gradient come through the scalar
  // unit, one load per wavefront instead of one per lane
  const uint32_t r0 = __builtin_amdgcn_readfirstlane(r);
  int64_t label;
  float g;
  if (__builtin_amdgcn_ballot_w64(r != r0) == 0) {
    label = labels[r0];
    g = Cvt<T>::load(grad_loss + r0);
  } else {
    label = labels[r];
    g = Cvt<T>::load(grad_loss + r);
  }
  // position of the label inside this vector, or a value no j reaches (labels outside the shard, negative ones)
  const uint64_t rel = uint64_t(label) - uint64_t(vocab_start) - uint64_t(c0);
  const uint32_t hit = rel < uint64_t(VEC) ? uint32_t(rel) : 0xffffffffu;
  float f[VEC];
  VecIO<T>::unpack(raw, f);
#pragma unroll
  for (int j = 0; j < VEC; ++j) f[j] = (uint32_t(j) == hit ? f[j] - 1.0f : f[j]) * g;
  st16_stream(out + size_t(v) * VEC, VecIO<T>::pack(f));
}

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void vocab_ce_bwd_scalar_kernel(const T* softmax, const int64_t* __restrict__ labels,
                                const T* __restrict__ grad_loss, T* out, int64_t total, int64_t cols,
                                int64_t vocab_start) {
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t r = i / cols;
  const uint64_t c = uint64_t(i - r * cols);
  const uint64_t hit = uint64_t(labels[r]) - uint64_t(vocab_start);
  const CT s = CT(Cvt<T>::load(softmax + i)), g = CT(Cvt<T>::load(grad_loss + r));
  Cvt<T>::store(out + i, (c == hit ? s - CT(1) : s) * g);
}

// ---------------------------------------------------------------------------
// The fused form: one read of the shard in the forward (hk_vocab_parallel_ce_stats, in the cross-entropy
// source), a per-row combination of the shards' statistics, and a backward that rebuilds softmax from the
// logits and the global log-sum-exp instead of reading a stored softmax.
// ---------------------------------------------------------------------------
// stats: [nshards, 3, rows] (maximum, sum of exp(x - maximum), picked logit) as an all-gather leaves them.
// lse[r] = log sum_k exp over the whole row; loss[r] = lse - picked logit, 0 for an ignored row.
template <typename T>
__global__ __launch_bounds__(256)
void vocab_ce_combine_kernel(const float* __restrict__ stats, int nshards, const int64_t* __restrict__ labels,
                             int64_t ignored_index, T* __restrict__ loss, float* __restrict__ lse, int64_t rows) {
  const int64_t r = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (r >= rows) return;
  float gmax = -__builtin_huge_valf();
  for (int k = 0; k < nshards; ++k) gmax = fmaxf(gmax, stats[(int64_t(k) * 3 + 0) * rows + r]);
  float gsum = 0.f, picked = 0.f;
  for (int k = 0; k < nshards; ++k) {
    const float m = stats[(int64_t(k) * 3 + 0) * rows + r];
    const float s = stats[(int64_t(k) * 3 + 1) * rows + r];
    if (s > 0.f) gsum += s * expf(m - gmax);
    picked += stats[(int64_t(k) * 3 + 2) * rows + r];
  }
  const bool ignored = labels[r] == ignored_index;
  const float l = ignored ? 0.f : logf(gsum) + gmax;
  if (lse) lse[r] = l;
  if (loss) {
    using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
    Cvt<T>::store(loss + r, CT(ignored ? 0.f : l - picked));
  }
}

// out[r, c] = (exp(x[r, c] - lse[r]) - [c == labels[r] - vocab_start]) * grad_loss[r]; zeros for an ignored row
template <typename T>
__global__ __launch_bounds__(kStreamThreads)
void vocab_ce_bwd_fused_kernel(const T* x, const int64_t* __restrict__ labels, const float* __restrict__ lse,
                               const T* __restrict__ grad_loss, T* out, uint32_t nvec, uint32_t cols_vec,
                               int64_t vocab_start, int64_t ignored_index) {
  constexpr int VEC = VecIO<T>::N;
  constexpr float kLog2e = 1.4426950408889634f;
  const uint32_t v = blockIdx.x * uint32_t(kStreamThreads) + threadIdx.x;
  if (v >= nvec) return;
  const uint32_t r = v / cols_vec;
  const uint32_t c0 = (v - r * cols_vec) * VEC;
  // all four loads are issued before any is waited for; an ignored row is read like the others (a branch on
  // the label around the vector load would put the two loads in series) and its result replaced by zeros
  const u32x4 raw = ld16(x + size_t(v) * VEC);
  // a wavefront almost always lies inside one row: then the row's three values come through the scalar unit,
  // one load per wavefront instead of one per lane
  const uint32_t r0 = __builtin_amdgcn_readfirstlane(r);
  int64_t label;
  float l2, g;
  if (__builtin_amdgcn_ballot_w64(r != r0) == 0) {
    label = labels[r0];
    l2 = lse[r0] * kLog2e;
    g = Cvt<T>::load(grad_loss + r0);
  } else {
    label = labels[r];
    l2 = lse[r] * kLog2e;
    g = Cvt<T>::load(grad_loss + r);
  }
  const bool ignored = label == ignored_index;
  g = ignored ? 0.f : g;
  float f[VEC];
  VecIO<T>::unpack(raw, f);
  // position of the label inside this vector, or a value no j reaches (labels outside the shard, negative ones)
  const uint64_t rel = uint64_t(label) - uint64_t(vocab_start) - uint64_t(c0);
  const uint32_t hit = rel < uint64_t(VEC) ? uint32_t(rel) : 0xffffffffu;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const float p = __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -l2));
    const float o = (uint32_t(j) == hit) ? fmaf(p, g, -g) : p * g;
    f[j] = ignored ? 0.f : o;              // also when exp overflowed to inf or the logit was NaN
  }
  st16_stream(out + size_t(v) * VEC, VecIO<T>::pack(f));
}

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void vocab_ce_bwd_fused_scalar_kernel(const T* x, const int64_t* __restrict__ labels, const float* __restrict__ lse,
                                      const T* __restrict__ grad_loss, T* out, int64_t total, int64_t cols,
                                      int64_t vocab_start, int64_t ignored_index) {
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t r = i / cols;
  const int64_t label = labels[r];
  CT o = CT(0);
  if (label != ignored_index) {
    const uint64_t hit = uint64_t(label) - uint64_t(vocab_start);
    const CT g = CT(Cvt<T>::load(grad_loss + r));
    const CT p = CT(exp(double(Cvt<T>::load(x + i)) - double(lse[r])));
    o = (uint64_t(i - r * cols) == hit) ? p * g - g : p * g;
  }
  Cvt<T>::store(out + i, o);
}

template <typename T>
static int vocab_bwd_fused_typed(const void* x, const int64_t* labels, const float* lse, const void* grad_loss,
                                 void* out, int64_t rows, int64_t cols, int64_t vocab_start, int64_t ignored_index,
                                 hipStream_t s) {
  const int64_t total = rows * cols;
  if constexpr (!std::is_same<T, double>::value) {
    constexpr int VEC = VecIO<T>::N;
    if (cols % VEC == 0 && aligned16(x) && aligned16(out) && total / VEC < 0x7fffffffLL) {
      const uint32_t nvec = uint32_t(total / VEC);
      profile_before(s);
      HK_LAUNCH((vocab_ce_bwd_fused_kernel<T>), dim3((nvec + kStreamThreads - 1) / kStreamThreads), dim3(kStreamThreads), 0, s,
                         static_cast<const T*>(x), labels, lse, static_cast<const T*>(grad_loss), static_cast<T*>(out),
                         nvec, uint32_t(cols / VEC), vocab_start, ignored_index);
      profile_after(s);
      return launch_check("vocab_ce_bwd_fused_kernel");
    }
  }
  HK_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd_fused: output too large");
  using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  profile_before(s);
  HK_LAUNCH((vocab_ce_bwd_fused_scalar_kernel<T, CT>), dim3(unsigned((total + 255) / 256)), dim3(256), 0, s,
                     static_cast<const T*>(x), labels, lse, static_cast<const T*>(grad_loss), static_cast<T*>(out),
                     total, cols, vocab_start, ignored_index);
  profile_after(s);
  return launch_check("vocab_ce_bwd_fused_scalar_kernel");
}

template <typename T>
static int vocab_bwd_typed(const void* softmax, const int64_t* labels, const void* grad_loss, void* out,
                           int64_t rows, int64_t cols, int64_t vocab_start, hipStream_t s) {
  const int64_t total = rows * cols;
  if constexpr (!std::is_same<T, double>::value) {
    constexpr int VEC = VecIO<T>::N;
    if (cols % VEC == 0 && aligned16(softmax) && aligned16(out) && total / VEC < 0x7fffffffLL) {
      const uint32_t nvec = uint32_t(total / VEC);
      profile_before(s);
      HK_LAUNCH((vocab_ce_bwd_vec_kernel<T>), dim3((nvec + kStreamThreads - 1) / kStreamThreads), dim3(kStreamThreads), 0, s,
                         static_cast<const T*>(softmax), labels, static_cast<const T*>(grad_loss),
                         static_cast<T*>(out), nvec, uint32_t(cols / VEC), vocab_start);
      profile_after(s);
      return launch_check("vocab_ce_bwd_vec_kernel");
    }
  }
  HK_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd: output too large");
  using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  profile_before(s);
  HK_LAUNCH((vocab_ce_bwd_scalar_kernel<T, CT>), dim3(unsigned((total + 255) / 256)), dim3(256), 0, s,
                     static_cast<const T*>(softmax), labels, static_cast<const T*>(grad_loss), static_cast<T*>(out),
                     total, cols, vocab_start);
  profile_after(s);
  return launch_check("vocab_ce_bwd_scalar_kernel");
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_vocab_parallel_ce_gather(int dtype, const void* logits, const int64_t* labels, int64_t rows, int64_t cols,
                                int64_t vocab_start, int64_t vocab_end, int64_t ignored_index, void* picked,
                                void* lse, hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "hk_vocab_parallel_ce_gather: negative shape");
  if (rows == 0) return HK_OK;
  HK_REQUIRE(logits && labels && picked && lse, HK_ERR_INVALID, "hk_vocab_parallel_ce_gather: null input/output");
  HK_REQUIRE(vocab_end - vocab_start <= cols && vocab_end >= vocab_start, HK_ERR_INVALID,
             "hk_vocab_parallel_ce_gather: shard [%lld, %lld) is wider than the %lld columns held",
             (long long) vocab_start, (long long) vocab_end, (long long) cols);
  hipStream_t s = as_hip(stream);
  const dim3 grid(unsigned((rows + 255) / 256)), block(256);
#define HK_VCE_GATHER(T)                                                                                         \
  HK_LAUNCH((vocab_ce_gather_kernel<T>), grid, block, 0, s, static_cast<const T*>(logits), labels, rows, \
                     cols, vocab_start, vocab_end, ignored_index, static_cast<T*>(picked), static_cast<T*>(lse))
  switch (dtype) {
    case HK_FLOAT32: HK_VCE_GATHER(float); break;
    case HK_BFLOAT16: HK_VCE_GATHER(bf16); break;
    case HK_FLOAT16: HK_VCE_GATHER(fp16); break;
    case HK_FLOAT64: HK_VCE_GATHER(double); break;
    default:
      set_last_error("hk_vocab_parallel_ce_gather: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_VCE_GATHER
  return launch_check("vocab_ce_gather_kernel");
}

int hk_vocab_parallel_ce_combine(int loss_dtype, const float* stats, int nshards, const int64_t* labels,
                                 int64_t ignored_index, void* loss, float* lse, int64_t rows, hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && nshards >= 1, HK_ERR_INVALID, "hk_vocab_parallel_ce_combine: bad shape");
  if (rows == 0) return HK_OK;
  HK_REQUIRE(stats && labels && (loss || lse), HK_ERR_INVALID, "hk_vocab_parallel_ce_combine: null input/output");
  hipStream_t s = as_hip(stream);
  const dim3 grid(unsigned((rows + 255) / 256)), block(256);
#define HK_VCE_COMBINE(T)                                                                                       \
  HK_LAUNCH((vocab_ce_combine_kernel<T>), grid, block, 0, s, stats, nshards, labels, ignored_index,    \
                     static_cast<T*>(loss), lse, rows)
  switch (loss_dtype) {
    case HK_FLOAT32: HK_VCE_COMBINE(float); break;
    case HK_BFLOAT16: HK_VCE_COMBINE(bf16); break;
    case HK_FLOAT16: HK_VCE_COMBINE(fp16); break;
    case HK_FLOAT64: HK_VCE_COMBINE(double); break;
    default:
      set_last_error("hk_vocab_parallel_ce_combine: not implemented for dtype %d", loss_dtype);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_VCE_COMBINE
  return launch_check("vocab_ce_combine_kernel");
}

int hk_vocab_parallel_ce_bwd_fused(int dtype, const void* logits, const int64_t* labels, const float* lse,
                                   const void* grad_loss, void* out, int64_t rows, int64_t cols,
                                   int64_t vocab_start, int64_t ignored_index, hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd_fused: negative shape");
  if (rows == 0 || cols == 0) return HK_OK;
  HK_REQUIRE(logits && labels && lse && grad_loss && out, HK_ERR_INVALID,
             "hk_vocab_parallel_ce_bwd_fused: null input/output");
  hipStream_t s = as_hip(stream);
#define HK_VCE_BWD(T) \
  return vocab_bwd_fused_typed<T>(logits, labels, lse, grad_loss, out, rows, cols, vocab_start, ignored_index, s)
  switch (dtype) {
    case HK_FLOAT32: HK_VCE_BWD(float);
    case HK_BFLOAT16: HK_VCE_BWD(bf16);
    case HK_FLOAT16: HK_VCE_BWD(fp16);
    case HK_FLOAT64: HK_VCE_BWD(double);
    default:
      set_last_error("hk_vocab_parallel_ce_bwd_fused: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_VCE_BWD
}

int hk_vocab_parallel_ce_bwd(int dtype, const void* softmax, const int64_t* labels, const void* grad_loss,
                             void* out, int64_t rows, int64_t cols, int64_t vocab_start, hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd: negative shape");
  if (rows == 0 || cols == 0) return HK_OK;
  HK_REQUIRE(softmax && labels && grad_loss && out, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd: null input/output");
  hipStream_t s = as_hip(stream);
  switch (dtype) {
    case HK_FLOAT32: return vocab_bwd_typed<float>(softmax, labels, grad_loss, out, rows, cols, vocab_start, s);
    case HK_BFLOAT16: return vocab_bwd_typed<bf16>(softmax, labels, grad_loss, out, rows, cols, vocab_start, s);
    case HK_FLOAT16: return vocab_bwd_typed<fp16>(softmax, labels, grad_loss, out, rows, cols, vocab_start, s);
    case HK_FLOAT64: return vocab_bwd_typed<double>(softmax, labels, grad_loss, out, rows, cols, vocab_start, s);
    default:
      set_last_error("hk_vocab_parallel_ce_bwd: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

} // extern "C"
