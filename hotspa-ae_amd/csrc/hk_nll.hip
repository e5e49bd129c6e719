// Negative log-likelihood loss on log-probabilities with int64 class labels, for gfx950.
//   forward   loss[r] = -pred[r, label[r]]                 (0 when the label is outside [0, cols))
//   backward  out[r, c] = (c == label[r]) ? -grad_loss[r] * cols : 0
// The forward is a gather of one element per row.  The backward writes every element of the output
// exactly once: the zero fill and the scatter are one pass of 128-bit stores, where the reference clears
// the array and then scatters in a second kernel (hetu/impl/kernel/NLLLoss.cu:8-41, :88-128).
#include "hk_common.h"

namespace hk {

template <typename T>
__global__ __launch_bounds__(256)
void nll_fwd_kernel(const T* pred, const int64_t* label, T* loss, int64_t rows, int64_t cols) {
  const int64_t r = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const int64_t id = label[r];
  float v = 0.f;
  if (id >= 0 && id < cols) v = -float(Cvt<T>::load(pred + r * cols + id));
  Cvt<T>::store(loss + r, v);
}

template <>
__global__ __launch_bounds__(256)
void nll_fwd_kernel<double>(const double* pred, const int64_t* label, double* loss, int64_t rows, int64_t cols) {
  const int64_t r = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const int64_t id = label[r];
  loss[r] = (id >= 0 && id < cols) ? -pred[r * cols + id] : 0.0;
}

// one 16-byte vector of the output per thread; VEC elements of T
template <typename T>
__global__ __launch_bounds__(256)
void nll_bwd_vec_kernel(const int64_t* label, const T* grad_loss, T* out, int64_t rows, int64_t cols,
                        int64_t nvec_row, float scale) {
  constexpr int VEC = VecIO<T>::N;
  const int64_t v = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (v >= rows * nvec_row) return;
  const int64_t r = v / nvec_row;
  const int64_t c0 = (v - r * nvec_row) * VEC;
  const int64_t id = label[r];
  float f[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) f[j] = 0.f;
  if (id >= c0 && id < c0 + VEC) {
    const float g = -Cvt<T>::load(grad_loss + r) * scale;
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = (c0 + j == id) ? g : 0.f;
  }
  st16_stream(out + r * cols + c0, VecIO<T>::pack(f));
}

// any alignment / width / dtype: one element per thread
template <typename T, typename CT>
__global__ __launch_bounds__(256)
void nll_bwd_scalar_kernel(const int64_t* label, const T* grad_loss, T* out, int64_t rows, int64_t cols, CT scale) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  const int64_t r = i / cols, c = i - r * cols;
  CT v = CT(0);
  if (label[r] == c) {
    if constexpr (std::is_same<T, double>::value) v = -grad_loss[r] * scale;
    else v = -CT(Cvt<T>::load(grad_loss + r)) * scale;
  }
  if constexpr (std::is_same<T, double>::value) out[i] = v;
  else Cvt<T>::store(out + i, float(v));
}

template <typename T>
static int nll_bwd_typed(const int64_t* label, const void* grad_loss, void* out, int64_t rows, int64_t cols,
                         hipStream_t s) {
  constexpr int VEC = 16 / int(sizeof(T));
  const int64_t total = rows * cols;
  if constexpr (!std::is_same<T, double>::value) {
    if (cols % VEC == 0 && aligned16(out)) {
      const int64_t nvec = total / VEC;
      HK_REQUIRE((nvec + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_nll_loss_bwd: output too large");
      profile_before(s);
      HK_LAUNCH((nll_bwd_vec_kernel<T>), dim3(unsigned((nvec + 255) / 256)), dim3(256), 0, s, label,
                         static_cast<const T*>(grad_loss), static_cast<T*>(out), rows, cols, cols / VEC, float(cols));
      profile_after(s);
      return launch_check("nll_bwd_vec_kernel");
    }
  }
  HK_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_nll_loss_bwd: output too large");
  using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  HK_LAUNCH((nll_bwd_scalar_kernel<T, CT>), dim3(unsigned((total + 255) / 256)), dim3(256), 0, s, label,
                     static_cast<const T*>(grad_loss), static_cast<T*>(out), rows, cols, CT(cols));
  return launch_check("nll_bwd_scalar_kernel");
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_nll_loss_fwd(int dtype, const void* pred, const int64_t* labels, void* loss, int64_t rows, int64_t cols,
                    hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "hk_nll_loss_fwd: negative shape");
  if (rows == 0) return HK_OK;
  HK_REQUIRE(pred && labels && loss, HK_ERR_INVALID, "hk_nll_loss_fwd: null input/output");
  HK_REQUIRE((rows + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_nll_loss_fwd: too many rows");
  hipStream_t s = as_hip(stream);
  const dim3 grid(unsigned((rows + 255) / 256)), block(256);
  profile_before(s);
  switch (dtype) {
    case HK_FLOAT32:
      HK_LAUNCH((nll_fwd_kernel<float>), grid, block, 0, s, static_cast<const float*>(pred), labels,
                         static_cast<float*>(loss), rows, cols);
      break;
    case HK_BFLOAT16:
      HK_LAUNCH((nll_fwd_kernel<bf16>), grid, block, 0, s, static_cast<const bf16*>(pred), labels,
                         static_cast<bf16*>(loss), rows, cols);
      break;
    case HK_FLOAT16:
      HK_LAUNCH((nll_fwd_kernel<fp16>), grid, block, 0, s, static_cast<const fp16*>(pred), labels,
                         static_cast<fp16*>(loss), rows, cols);
      break;
    case HK_FLOAT64:
      HK_LAUNCH((nll_fwd_kernel<double>), grid, block, 0, s, static_cast<const double*>(pred), labels,
                         static_cast<double*>(loss), rows, cols);
      break;
    default:
      set_last_error("hk_nll_loss_fwd: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
  profile_after(s);
  return launch_check("nll_fwd_kernel");
}

int hk_nll_loss_bwd(int dtype, const int64_t* labels, const void* grad_loss, void* out, int64_t rows,
                    int64_t cols, hkStream_t stream) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "hk_nll_loss_bwd: negative shape");
  if (rows == 0 || cols == 0) return HK_OK;
  HK_REQUIRE(labels && grad_loss && out, HK_ERR_INVALID, "hk_nll_loss_bwd: null input/output");
  hipStream_t s = as_hip(stream);
  switch (dtype) {
    case HK_FLOAT32: return nll_bwd_typed<float>(labels, grad_loss, out, rows, cols, s);
    case HK_BFLOAT16: return nll_bwd_typed<bf16>(labels, grad_loss, out, rows, cols, s);
    case HK_FLOAT16: return nll_bwd_typed<fp16>(labels, grad_loss, out, rows, cols, s);
    case HK_FLOAT64: return nll_bwd_typed<double>(labels, grad_loss, out, rows, cols, s);
    default:
      set_last_error("hk_nll_loss_bwd: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

} // extern "C"
