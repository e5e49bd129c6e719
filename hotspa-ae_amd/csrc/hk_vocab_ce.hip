// Local kernels of the vocabulary-parallel cross-entropy: every device holds the
// columns [vocab_start, vocab_end) of the logits; what crosses devices (the row
// maximum, the sum of exponentials, the picked logit) is reduced by the caller
// between these kernels.
#include "hk_common.cuh"

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
__global__ __launch_bounds__(256)
void vocab_ce_bwd_vec_kernel(const T* softmax, const int64_t* __restrict__ labels, const T* __restrict__ grad_loss,
                             T* out, int64_t nvec, int64_t cols_vec, int64_t vocab_start) {
  constexpr int VEC = VecIO<T>::N;
  const int64_t v = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (v >= nvec) return;
  const int64_t r = v / cols_vec;
  const int64_t c0 = (v - r * cols_vec) * VEC;
  const uint64_t hit = uint64_t(labels[r]) - uint64_t(vocab_start);
  const float g = Cvt<T>::load(grad_loss + r);
  float f[VEC];
  VecIO<T>::unpack(ld16(softmax + v * VEC), f);
#pragma unroll
  for (int j = 0; j < VEC; ++j) f[j] = (uint64_t(c0 + j) == hit ? f[j] - 1.0f : f[j]) * g;
  st16_stream(out + v * VEC, VecIO<T>::pack(f));
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

template <typename T>
static int vocab_bwd_typed(const void* softmax, const int64_t* labels, const void* grad_loss, void* out,
                           int64_t rows, int64_t cols, int64_t vocab_start, hipStream_t s) {
  const int64_t total = rows * cols;
  if constexpr (!std::is_same<T, double>::value) {
    constexpr int VEC = VecIO<T>::N;
    if (cols % VEC == 0 && aligned16(softmax) && aligned16(out)) {
      const int64_t nvec = total / VEC;
      HK_REQUIRE((nvec + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd: output too large");
      profile_before(s);
      hipLaunchKernelGGL((vocab_ce_bwd_vec_kernel<T>), dim3(unsigned((nvec + 255) / 256)), dim3(256), 0, s,
                         static_cast<const T*>(softmax), labels, static_cast<const T*>(grad_loss),
                         static_cast<T*>(out), nvec, cols / VEC, vocab_start);
      profile_after(s);
      return launch_check("vocab_ce_bwd_vec_kernel");
    }
  }
  HK_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_vocab_parallel_ce_bwd: output too large");
  using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  profile_before(s);
  hipLaunchKernelGGL((vocab_ce_bwd_scalar_kernel<T, CT>), dim3(unsigned((total + 255) / 256)), dim3(256), 0, s,
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
  hipLaunchKernelGGL((vocab_ce_gather_kernel<T>), grid, block, 0, s, static_cast<const T*>(logits), labels, rows, \
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
