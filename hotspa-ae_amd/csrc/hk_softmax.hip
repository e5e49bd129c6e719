// Softmax forward / backward for gfx950.
//
// Last-dimension softmax keeps the row in registers (one HBM read, one write):
// every thread folds its elements into a (max, sum-of-exp) pair, the pairs are
// merged online across lanes (DPP) and waves (LDS), and the stored exponentials
// are rescaled on the way out, so exp is evaluated once per element.
// One wavefront per row for short rows, one workgroup per row for long rows.
#include "hk_common.h"

#include <algorithm>

namespace hk {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -__builtin_huge_valf();

struct SoftmaxArgs {
  const void* x;    // forward: input;  backward: y
  const void* dy;   // backward only
  void* out;        // forward: y;      backward: dx
  int64_t rows;
  int64_t x_pitch, dy_pitch, out_pitch;   // elements between row starts (== cols for a dense array)
  int64_t n0, n1, n2;                     // rows on several levels in walk order (see LevelSteps); one level: n0 = rows
  LevelSteps x_lv, dy_lv, out_lv;
  int cols;
  int nvec;
};

template <typename T, int NV, bool WAVE_ROW>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024)
void softmax_fwd_kernel(SoftmaxArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves * 2];
  const int tpr = WAVE_ROW ? kWave : int(blockDim.x);
  const int t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  const int64_t row = WAVE_ROW
      ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index()
      : int64_t(blockIdx.x);
  if (WAVE_ROW && row >= a.n0) return;   // row counts within the innermost level
  const int nwaves = WAVE_ROW ? 1 : int(blockDim.x >> 6);

  const T* xr = static_cast<const T*>(a.x) + row * a.x_pitch + outer_level_offset(a.x_lv);
  // slots past the row's end hold -inf: they change neither the maximum nor the sum
  u32x4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if ((i + 1) * tpr <= a.nvec) {       // uniform: every thread's slot i is inside the row
      raw[i] = ld16(xr + v * VEC);
    } else {
      raw[i] = neg_inf_vec<T>();
      if (v < a.nvec) raw[i] = ld16(xr + v * VEC);
    }
  }
  float e[NV * VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i) VecIO<T>::unpack(raw[i], &e[i * VEC]);
  static_assert((NV * VEC) % 2 == 0, "pairs of elements per max3");
  float m = fmaxf(e[0], e[1]);
#pragma unroll
  for (int k = 2; k < NV * VEC; k += 2) m = max3(m, e[k], e[k + 1]);
  // ml: this thread's maximum in the log2 domain, rounded once (see OnlineSoftmaxTuple)
  const float ml = (m == kNegInf) ? 0.f : m * kLog2e;
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV * VEC; ++k) {
    e[k] = __builtin_amdgcn_exp2f(fmaf(e[k], kLog2e, -ml));
    s += e[k];
  }
  MaxSumTuple p;
  p.v[0] = (m == kNegInf) ? kNegInf : ml; p.v[1] = s;
  p = WAVE_ROW ? wave_allreduce_tuple(p) : group_allreduce_tuple(p, red, 0, nwaves);
  const float ML = (p.v[0] == kNegInf) ? 0.f : p.v[0];
  const float scale = __builtin_amdgcn_exp2f(ml - ML) / p.v[1];

  T* yr = static_cast<T*>(a.out) + row * a.out_pitch + outer_level_offset(a.out_lv);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if (v < a.nvec) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) e[i * VEC + j] *= scale;
      const u32x4 o = VecIO<T>::pack(&e[i * VEC]);
      st16_stream(yr + v * VEC, o);
    }
  }
}

template <typename T, int NV, bool WAVE_ROW>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024)
void softmax_bwd_kernel(SoftmaxArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves];
  const int tpr = WAVE_ROW ? kWave : int(blockDim.x);
  const int t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  const int64_t row = WAVE_ROW
      ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index()
      : int64_t(blockIdx.x);
  if (WAVE_ROW && row >= a.n0) return;   // row counts within the innermost level
  const int nwaves = WAVE_ROW ? 1 : int(blockDim.x >> 6);

  const T* yr = static_cast<const T*>(a.x) + row * a.x_pitch + outer_level_offset(a.x_lv);
  const T* dyr = static_cast<const T*>(a.dy) + row * a.dy_pitch + outer_level_offset(a.dy_lv);
  u32x4 ry[NV], rdy[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    ry[i] = u32x4{0, 0, 0, 0};
    rdy[i] = u32x4{0, 0, 0, 0};
    if (v < a.nvec) { ry[i] = ld16(yr + v * VEC); rdy[i] = ld16(dyr + v * VEC); }
  }
  SumTuple<1> s;
  s.v[0] = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    float y[VEC], d[VEC];
    VecIO<T>::unpack(ry[i], y);
    VecIO<T>::unpack(rdy[i], d);
#pragma unroll
    for (int j = 0; j < VEC; ++j) s.v[0] = fmaf(y[j], d[j], s.v[0]);  // padding is zero
  }
  s = WAVE_ROW ? wave_allreduce_tuple(s) : group_allreduce_tuple(s, red, 0, nwaves);
  const float dot = s.v[0];
  T* dxr = static_cast<T*>(a.out) + row * a.out_pitch + outer_level_offset(a.out_lv);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if (v < a.nvec) {
      float y[VEC], d[VEC];
      VecIO<T>::unpack(ry[i], y);
      VecIO<T>::unpack(rdy[i], d);
#pragma unroll
      for (int j = 0; j < VEC; ++j) d[j] = y[j] * (d[j] - dot);
      const u32x4 o = VecIO<T>::pack(d);
      st16_stream(dxr + v * VEC, o);
    }
  }
}

// Softmax along a dimension of extent `dim` with element stride `inner`
// (inner == 1: rows too long or too unaligned for the register kernels).
// One thread walks one (outer, inner) position, threads of a wave sit on
// neighbouring inner positions; for inner == 1 one workgroup takes one row.
template <typename T, typename CT>
struct SmIO {
  static __device__ __forceinline__ CT ld(const T* p) { return CT(Cvt<T>::load(p)); }
  static __device__ __forceinline__ void st(T* p, CT v) { Cvt<T>::store(p, v); }
};

template <typename CT> __device__ __forceinline__ CT exp_ct(CT v);
template <> __device__ __forceinline__ float exp_ct<float>(float v) { return __builtin_amdgcn_exp2f(v * kLog2e); }
template <> __device__ __forceinline__ double exp_ct<double>(double v) { return exp(v); }

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void softmax_fwd_strided_kernel(const T* x, T* y, int64_t outer, int64_t dim, int64_t inner) {
  const int64_t pos = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (pos >= outer * inner) return;
  const int64_t o = pos / inner, in = pos - o * inner;
  const T* xp = x + o * dim * inner + in;
  T* yp = y + o * dim * inner + in;
  CT m = -__builtin_huge_val(), s = 0;
  for (int64_t k = 0; k < dim; ++k) {
    const CT v = SmIO<T, CT>::ld(xp + k * inner);
    m = v > m ? v : m;
  }
  for (int64_t k = 0; k < dim; ++k) s += exp_ct<CT>(SmIO<T, CT>::ld(xp + k * inner) - m);
  const CT inv = CT(1) / s;
  for (int64_t k = 0; k < dim; ++k)
    SmIO<T, CT>::st(yp + k * inner, exp_ct<CT>(SmIO<T, CT>::ld(xp + k * inner) - m) * inv);
}

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void softmax_bwd_strided_kernel(const T* y, const T* dy, T* dx, int64_t outer, int64_t dim,
                                int64_t inner) {
  const int64_t pos = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (pos >= outer * inner) return;
  const int64_t o = pos / inner, in = pos - o * inner;
  const int64_t base = o * dim * inner + in;
  CT dot = 0;
  for (int64_t k = 0; k < dim; ++k)
    dot += SmIO<T, CT>::ld(y + base + k * inner) * SmIO<T, CT>::ld(dy + base + k * inner);
  for (int64_t k = 0; k < dim; ++k) {
    const CT yv = SmIO<T, CT>::ld(y + base + k * inner);
    SmIO<T, CT>::st(dx + base + k * inner, yv * (SmIO<T, CT>::ld(dy + base + k * inner) - dot));
  }
}

template <typename CT>
__device__ __forceinline__ CT block_reduce_generic(CT v, CT* lds, bool is_max) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
    if (tid < s) lds[tid] = is_max ? (lds[tid] > lds[tid + s] ? lds[tid] : lds[tid + s])
                                   : lds[tid] + lds[tid + s];
    __syncthreads();
  }
  CT r = lds[0];
  __syncthreads();
  return r;
}

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void softmax_fwd_longrow_kernel(const T* x, T* y, int64_t cols, int64_t x_pitch, int64_t y_pitch) {
  __shared__ CT lds[256];
  const T* xr = x + int64_t(blockIdx.x) * x_pitch;
  T* yr = y + int64_t(blockIdx.x) * y_pitch;
  CT m = -__builtin_huge_val();
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
    const CT v = SmIO<T, CT>::ld(xr + c);
    m = v > m ? v : m;
  }
  m = block_reduce_generic<CT>(m, lds, true);
  CT s = 0;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) s += exp_ct<CT>(SmIO<T, CT>::ld(xr + c) - m);
  s = block_reduce_generic<CT>(s, lds, false);
  const CT inv = CT(1) / s;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x)
    SmIO<T, CT>::st(yr + c, exp_ct<CT>(SmIO<T, CT>::ld(xr + c) - m) * inv);
}

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void softmax_bwd_longrow_kernel(const T* y, const T* dy, T* dx, int64_t cols, int64_t y_pitch,
                                int64_t dy_pitch, int64_t dx_pitch) {
  __shared__ CT lds[256];
  const T* yr = y + int64_t(blockIdx.x) * y_pitch;
  const T* dyr = dy + int64_t(blockIdx.x) * dy_pitch;
  T* dxr = dx + int64_t(blockIdx.x) * dx_pitch;
  CT dot = 0;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x)
    dot += SmIO<T, CT>::ld(yr + c) * SmIO<T, CT>::ld(dyr + c);
  dot = block_reduce_generic<CT>(dot, lds, false);
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
    const CT yv = SmIO<T, CT>::ld(yr + c);
    SmIO<T, CT>::st(dxr + c, yv * (SmIO<T, CT>::ld(dyr + c) - dot));
  }
}

static inline int pow2_ceil_sm(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// threads per row / vectors per thread for a row of nvec 16-byte vectors
static bool pick_softmax_shape(int nvec, int max_nv_wave, int max_nv, bool bwd, int* threads, int* nv) {
  const int forced = tune_get(TUNE_SOFTMAX_THREADS);
  if (forced > 0) {
    int t = std::min(1024, std::max(64, (forced + 63) / 64 * 64));
    int n = pow2_ceil_sm((nvec + t - 1) / t);
    if (n > max_nv) return false;
    *threads = t; *nv = n;
    return true;
  }
  // measured on MI355X at 2048 bf16 columns: forward is fastest with two
  // vectors per thread (128 threads per row), backward with one (256 threads)
  const int want = bwd ? 1 : 2;
  if (nvec <= 64 * want) {
    *threads = 64;
    *nv = pow2_ceil_sm((nvec + 63) / 64);
    return *nv <= max_nv_wave;
  }
  for (int n = want; n <= max_nv; n <<= 1) {
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 1024) { *threads = t; *nv = n; return true; }
  }
  return false;
}

template <typename T, bool BWD, bool WAVE_ROW>
static int launch_softmax_nv(const SoftmaxArgs& a, int nv, dim3 grid, dim3 block, hipStream_t s) {
#define HK_SM_CASE(N)                                                                      \
  case N:                                                                                  \
    if constexpr (BWD) HK_LAUNCH((softmax_bwd_kernel<T, N, WAVE_ROW>), grid, block, 0, s, a); \
    else HK_LAUNCH((softmax_fwd_kernel<T, N, WAVE_ROW>), grid, block, 0, s, a);   \
    break;
  profile_before(s);
  switch (nv) {
    HK_SM_CASE(1) HK_SM_CASE(2) HK_SM_CASE(4) HK_SM_CASE(8)
    case 16:
      if constexpr (VecIO<T>::N == 4 && !BWD) {
        HK_LAUNCH((softmax_fwd_kernel<T, 16, WAVE_ROW>), grid, block, 0, s, a);
        break;
      }
      [[fallthrough]];
    default:
      set_last_error("softmax: no kernel for %d vectors per thread", nv);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_SM_CASE
  profile_after(s);
  return launch_check(BWD ? "softmax_bwd_kernel" : "softmax_fwd_kernel");
}

template <typename T, bool BWD>
static int softmax_lastdim_typed(SoftmaxArgs a, hipStream_t s) {
  constexpr int VEC = VecIO<T>::N;
  auto steps_ok = [](int64_t pitch, const LevelSteps& l) { return pitch % VEC == 0 && l.p1 % VEC == 0 && l.p2 % VEC == 0; };
  const bool vec_ok = a.cols % VEC == 0 && aligned16(a.x) && aligned16(a.dy) && aligned16(a.out) &&
                      steps_ok(a.x_pitch, a.x_lv) && steps_ok(a.out_pitch, a.out_lv) &&
                      (!BWD || steps_ok(a.dy_pitch, a.dy_lv));
  a.nvec = a.cols / VEC;
  // forward keeps NV*VEC exponentials per thread: at most 64 floats
  // backward holds y and dy: at most 4 vectors of each per thread
  const int max_nv = BWD ? 4 : 64 / VEC;
  const int max_nv_wave = BWD ? 4 : std::min(8, 64 / VEC);
  int threads = 0, nv = 0;
  if (vec_ok && pick_softmax_shape(a.nvec, max_nv_wave, max_nv, BWD, &threads, &nv)) {
    if (threads == 64) {
      dim3 grid(unsigned((a.n0 + 3) / 4), unsigned(a.n1), unsigned(a.n2)), block(256);
      return launch_softmax_nv<T, BWD, true>(a, nv, grid, block, s);
    }
    dim3 grid{unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)}, block{unsigned(threads)};
    return launch_softmax_nv<T, BWD, false>(a, nv, grid, block, s);
  }
  if (a.n0 != a.rows) {
    set_last_error("softmax: rows on several levels need 16-byte aligned rows and steps");
    return HK_ERR_UNSUPPORTED;
  }
  if constexpr (BWD) {
    HK_LAUNCH((softmax_bwd_longrow_kernel<T, float>), dim3(unsigned(a.rows)), dim3(256), 0, s,
                       static_cast<const T*>(a.x), static_cast<const T*>(a.dy), static_cast<T*>(a.out),
                       int64_t(a.cols), a.x_pitch, a.dy_pitch, a.out_pitch);
    return launch_check("softmax_bwd_longrow_kernel");
  } else {
    HK_LAUNCH((softmax_fwd_longrow_kernel<T, float>), dim3(unsigned(a.rows)), dim3(256), 0, s,
                       static_cast<const T*>(a.x), static_cast<T*>(a.out), int64_t(a.cols), a.x_pitch, a.out_pitch);
    return launch_check("softmax_fwd_longrow_kernel");
  }
}

template <typename T, typename CT, bool BWD>
static int softmax_strided_typed(const void* x, const void* dy, void* out, int64_t outer, int64_t dim,
                                 int64_t inner, int64_t x_pitch, int64_t dy_pitch, int64_t out_pitch,
                                 hipStream_t s) {
  if (inner == 1) {
    if constexpr (BWD) {
      HK_LAUNCH((softmax_bwd_longrow_kernel<T, CT>), dim3(unsigned(outer)), dim3(256), 0, s,
                         static_cast<const T*>(x), static_cast<const T*>(dy), static_cast<T*>(out), dim, x_pitch,
                         dy_pitch, out_pitch);
    } else {
      HK_LAUNCH((softmax_fwd_longrow_kernel<T, CT>), dim3(unsigned(outer)), dim3(256), 0, s,
                         static_cast<const T*>(x), static_cast<T*>(out), dim, x_pitch, out_pitch);
    }
    return launch_check("softmax_longrow_kernel");
  }
  const int64_t npos = outer * inner;
  const int64_t blocks = (npos + 255) / 256;
  if constexpr (BWD) {
    HK_LAUNCH((softmax_bwd_strided_kernel<T, CT>), dim3(unsigned(blocks)), dim3(256), 0, s,
                       static_cast<const T*>(x), static_cast<const T*>(dy), static_cast<T*>(out), outer,
                       dim, inner);
  } else {
    HK_LAUNCH((softmax_fwd_strided_kernel<T, CT>), dim3(unsigned(blocks)), dim3(256), 0, s,
                       static_cast<const T*>(x), static_cast<T*>(out), outer, dim, inner);
  }
  return launch_check("softmax_strided_kernel");
}

// x_pitch / dy_pitch / out_pitch: elements between the starts of consecutive rows when inner == 1 (0: dense, the
// row's own length); a dimension other than the last (inner > 1) only exists for dense arrays.
struct SoftmaxLevels {
  int64_t n0, n1, n2;          // in walk order
  int64_t x_pitch, dy_pitch, out_pitch;
  LevelSteps x, dy, out;
};

template <bool BWD>
static int softmax_dispatch(int dtype, const void* x, const void* dy, void* out, int64_t outer,
                            int64_t dim, int64_t inner, int64_t x_pitch, int64_t dy_pitch, int64_t out_pitch,
                            hipStream_t s, const char* who, const SoftmaxLevels* levels = nullptr) {
  HK_REQUIRE(outer >= 0 && dim >= 0 && inner >= 0, HK_ERR_INVALID, "%s: negative extent", who);
  if (outer == 0 || dim == 0 || inner == 0) return HK_OK;
  HK_REQUIRE(x && out && (!BWD || dy), HK_ERR_INVALID, "%s: null input/output", who);
  if (x_pitch == 0) x_pitch = dim;
  if (dy_pitch == 0) dy_pitch = dim;
  if (out_pitch == 0) out_pitch = dim;
  HK_REQUIRE((levels && levels->n0 == 1) || (x_pitch >= dim && out_pitch >= dim && dy_pitch >= dim), HK_ERR_INVALID,
             "%s: a row pitch is smaller than the %lld columns of a row", who, (long long)dim);
  HK_REQUIRE(inner == 1 || (x_pitch == dim && dy_pitch == dim && out_pitch == dim), HK_ERR_INVALID,
             "%s: row pitches only apply to the last dimension", who);
  HK_REQUIRE(outer <= 0x7fffffffLL && (outer * inner + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID,
             "%s: too many rows", who);
  if (inner == 1 && dim <= 0x3fffffff && dtype != HK_FLOAT64) {
    SoftmaxArgs a{};
    a.x = x; a.dy = dy; a.out = out; a.rows = outer; a.cols = int(dim);
    a.x_pitch = x_pitch; a.dy_pitch = dy_pitch; a.out_pitch = out_pitch;
    a.n0 = outer; a.n1 = a.n2 = 1;
    if (levels) {
      a.n0 = levels->n0; a.n1 = levels->n1; a.n2 = levels->n2;
      a.x_lv = levels->x; a.dy_lv = levels->dy; a.out_lv = levels->out;
    }
    switch (dtype) {
      case HK_FLOAT32: return softmax_lastdim_typed<float, BWD>(a, s);
      case HK_BFLOAT16: return softmax_lastdim_typed<bf16, BWD>(a, s);
      case HK_FLOAT16: return softmax_lastdim_typed<fp16, BWD>(a, s);
      default: break;
    }
  }
  if (levels && levels->n0 != outer) {
    set_last_error("%s: rows on several levels are not implemented for dtype %d", who, dtype);
    return HK_ERR_UNSUPPORTED;
  }
  switch (dtype) {
    case HK_FLOAT32: return softmax_strided_typed<float, float, BWD>(x, dy, out, outer, dim, inner, x_pitch, dy_pitch, out_pitch, s);
    case HK_BFLOAT16: return softmax_strided_typed<bf16, float, BWD>(x, dy, out, outer, dim, inner, x_pitch, dy_pitch, out_pitch, s);
    case HK_FLOAT16: return softmax_strided_typed<fp16, float, BWD>(x, dy, out, outer, dim, inner, x_pitch, dy_pitch, out_pitch, s);
    case HK_FLOAT64: return softmax_strided_typed<double, double, BWD>(x, dy, out, outer, dim, inner, x_pitch, dy_pitch, out_pitch, s);
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_softmax_fwd(int dtype, const void* x, void* y, int64_t outer, int64_t dim, int64_t inner,
                   hkStream_t stream) {
  return softmax_dispatch<false>(dtype, x, nullptr, y, outer, dim, inner, 0, 0, 0, as_hip(stream), "hk_softmax_fwd");
}

int hk_softmax_fwd_pitched(int dtype, const void* x, int64_t x_pitch, void* y, int64_t y_pitch, int64_t rows,
                           int64_t cols, hkStream_t stream) {
  HK_REQUIRE(x_pitch > 0 && y_pitch > 0, HK_ERR_INVALID, "hk_softmax_fwd_pitched: a row pitch must be positive");
  return softmax_dispatch<false>(dtype, x, nullptr, y, rows, cols, 1, x_pitch, x_pitch, y_pitch, as_hip(stream),
                                 "hk_softmax_fwd_pitched");
}

static int softmax_levels(const int64_t level_rows[3], const int64_t* x_steps, const int64_t* dy_steps,
                          const int64_t* out_steps, SoftmaxLevels* lv, int64_t* rows, const char* who) {
  HK_REQUIRE(level_rows && x_steps && out_steps, HK_ERR_INVALID, "%s: null level_rows / steps", who);
  const int64_t n0 = level_rows[0], n1 = level_rows[1], n2 = level_rows[2];
  HK_REQUIRE(n0 >= 0 && n1 >= 0 && n2 >= 0, HK_ERR_INVALID, "%s: negative level count", who);
  *rows = 0;
  if (n0 == 0 || n1 == 0 || n2 == 0) return HK_OK;
  HK_REQUIRE(n0 <= 0x7fffffffLL && n0 * n1 <= 0x7fffffffLL && n0 * n1 * n2 <= 0x7fffffffLL, HK_ERR_INVALID,
             "%s: too many rows", who);
  *rows = n0 * n1 * n2;
  int64_t key[3] = {0, 0, 0};
  for (int k = 0; k < 3; ++k) key[k] = x_steps[k] + out_steps[k] + (dy_steps ? dy_steps[k] : 0);
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  HK_REQUIRE(walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)n0, (long long)n1, (long long)n2);
  lv->n0 = w.n[0]; lv->n1 = w.n[1]; lv->n2 = w.n[2];
  walk_steps(w, x_steps, &lv->x_pitch, &lv->x);
  walk_steps(w, out_steps, &lv->out_pitch, &lv->out);
  lv->dy_pitch = lv->x_pitch;
  lv->dy = lv->x;
  if (dy_steps) walk_steps(w, dy_steps, &lv->dy_pitch, &lv->dy);
  return HK_OK;
}

int hk_softmax_fwd_strided_rows(int dtype, const void* x, const int64_t x_steps[3], void* y, const int64_t y_steps[3],
                                const int64_t level_rows[3], int64_t cols, hkStream_t stream) {
  const char* who = "hk_softmax_fwd_strided_rows";
  SoftmaxLevels lv{};
  int64_t rows = 0;
  int rc = softmax_levels(level_rows, x_steps, nullptr, y_steps, &lv, &rows, who);
  if (rc != HK_OK || rows == 0) return rc;
  return softmax_dispatch<false>(dtype, x, nullptr, y, rows, cols, 1, lv.x_pitch, lv.dy_pitch, lv.out_pitch,
                                 as_hip(stream), who, &lv);
}

int hk_softmax_bwd_strided_rows(int dtype, const void* y, const int64_t y_steps[3], const void* dy,
                                const int64_t dy_steps[3], void* dx, const int64_t dx_steps[3],
                                const int64_t level_rows[3], int64_t cols, hkStream_t stream) {
  const char* who = "hk_softmax_bwd_strided_rows";
  HK_REQUIRE(dy_steps, HK_ERR_INVALID, "%s: null steps", who);
  SoftmaxLevels lv{};
  int64_t rows = 0;
  int rc = softmax_levels(level_rows, y_steps, dy_steps, dx_steps, &lv, &rows, who);
  if (rc != HK_OK || rows == 0) return rc;
  return softmax_dispatch<true>(dtype, y, dy, dx, rows, cols, 1, lv.x_pitch, lv.dy_pitch, lv.out_pitch,
                                as_hip(stream), who, &lv);
}

int hk_softmax_bwd(int dtype, const void* y, const void* dy, void* dx, int64_t outer, int64_t dim,
                   int64_t inner, hkStream_t stream) {
  return softmax_dispatch<true>(dtype, y, dy, dx, outer, dim, inner, 0, 0, 0, as_hip(stream), "hk_softmax_bwd");
}

int hk_softmax_bwd_pitched(int dtype, const void* y, int64_t y_pitch, const void* dy, int64_t dy_pitch, void* dx,
                           int64_t dx_pitch, int64_t rows, int64_t cols, hkStream_t stream) {
  HK_REQUIRE(y_pitch > 0 && dy_pitch > 0 && dx_pitch > 0, HK_ERR_INVALID,
             "hk_softmax_bwd_pitched: a row pitch must be positive");
  return softmax_dispatch<true>(dtype, y, dy, dx, rows, cols, 1, y_pitch, dy_pitch, dx_pitch, as_hip(stream),
                                "hk_softmax_bwd_pitched");
}

} // extern "C"
