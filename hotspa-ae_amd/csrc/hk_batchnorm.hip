// Spatial batch normalisation of an NCHW array in training mode, forward and
// backward, with the semantics of cuDNN's cudnnBatchNormalizationForwardTraining /
// cudnnBatchNormalizationBackward in CUDNN_BATCHNORM_SPATIAL mode (what the
// reference calls): per channel over N, H, W.
//
// A channel's data is N runs of H*W contiguous elements, C*H*W apart.  Three
// launches each way: (1) per-channel partial statistics from several workgroups
// per channel, (2) a one-thread-per-channel merge that also writes the saved /
// running statistics and the per-channel coefficients, (3) an element-wise pass,
// one 16-byte vector per thread.  The input is read twice and the output written
// once in the forward; the backward reads dy and x twice and writes dx once.
#include "hk_common.h"

#include <algorithm>
#include <type_traits>

namespace hk {

template <typename T> struct BnCT { using type = float; };
template <> struct BnCT<double> { using type = double; };

// V elements starting at p as compute-type values (V == 1: any alignment)
template <typename T, int V, typename CT>
__device__ __forceinline__ void bn_load(const T* p, CT* f) {
  if constexpr (V == 1) {
    f[0] = CT(Cvt<T>::load(p));
  } else {
    float t[V];
    VecIO<T>::unpack(ld16(p), t);
#pragma unroll
    for (int j = 0; j < V; ++j) f[j] = t[j];
  }
}
template <typename T, int V, typename CT>
__device__ __forceinline__ void bn_store(T* p, const CT* f) {
  if constexpr (V == 1) {
    Cvt<T>::store(p, f[0]);
  } else {
    float t[V];
#pragma unroll
    for (int j = 0; j < V; ++j) t[j] = f[j];
    st16_stream(p, VecIO<T>::pack(t));
  }
}

struct BnShape {
  int64_t N, C, HW;
  int64_t hw_vec;         // HW / V
  int64_t per_channel;    // N * hw_vec: loads of V elements per channel
  int splits;
};

// A thread's walk over the loads v0, v0 + stride, v0 + 2 stride, ... (< per_channel) of channel c: the element
// offset of the current load, kept up by additions (one division per thread at the start, none per load).
struct BnWalk {
  int64_t off;        // element offset of the current load
  int64_t in_plane;   // its load index inside its H*W plane
  int64_t left;       // loads still to do, the current one included
  int64_t step_off, step_in_plane, wrap_off, hw_vec;
  __device__ __forceinline__ BnWalk(const BnShape& s, int64_t c, int64_t v0, int64_t stride, int V) {
    const int64_t n = v0 / s.hw_vec;
    in_plane = v0 - n * s.hw_vec;
    off = (n * s.C + c) * s.HW + in_plane * V;
    left = v0 < s.per_channel ? (s.per_channel - v0 + stride - 1) / stride : 0;
    const int64_t q = stride / s.hw_vec;                 // whole planes per step
    step_in_plane = stride - q * s.hw_vec;
    step_off = q * s.C * s.HW + step_in_plane * V;
    wrap_off = (s.C - 1) * s.HW;                         // from the end of a plane to the same channel of the next image
    hw_vec = s.hw_vec;
  }
  __device__ __forceinline__ void next() {
    in_plane += step_in_plane;
    off += step_off;
    const bool wrap = in_plane >= hw_vec;
    in_plane -= wrap ? hw_vec : 0;
    off += wrap ? wrap_off : 0;
    --left;
  }
};

template <typename CT>
__device__ __forceinline__ CT block_sum(CT v, CT* lds) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
    if (tid < s) lds[tid] += lds[tid + s];
    __syncthreads();
  }
  const CT r = lds[0];
  __syncthreads();
  return r;
}

// (count, mean, M2) of a slice of one channel -> part[(c * splits + split) * 3 ..]
template <typename T, int V, typename CT>
__global__ __launch_bounds__(256)
void bn_stats_kernel(const T* __restrict__ x, BnShape s, CT* __restrict__ part) {
  __shared__ CT lds[256];
  const int64_t c = blockIdx.x;
  const int split = blockIdx.y;
  // per thread: sums of (x - K) and (x - K)^2 about a pivot K taken from the thread's first load, so that a
  // large common offset of the channel never enters a sum; no division inside the loop
  BnWalk w(s, c, int64_t(split) * 256 + threadIdx.x, int64_t(s.splits) * 256, V);
  CT cnt = 0, mean = 0, m2 = 0;
  if (w.left > 0) {
    CT f[V];
    bn_load<T, V, CT>(x + w.off, f);
    CT K = 0;
#pragma unroll
    for (int j = 0; j < V; ++j) K += f[j];
    K /= CT(V);
    CT s1 = 0, s2 = 0;
#pragma unroll
    for (int j = 0; j < V; ++j) { const CT d = f[j] - K; s1 += d; s2 += d * d; }
    cnt = CT(V);
    for (w.next(); w.left > 0; w.next()) {
      bn_load<T, V, CT>(x + w.off, f);
#pragma unroll
      for (int j = 0; j < V; ++j) { const CT d = f[j] - K; s1 += d; s2 += d * d; }
      cnt += CT(V);
    }
    mean = K + s1 / cnt;
    m2 = s2 - s1 * (s1 / cnt);
    m2 = m2 > 0 ? m2 : CT(0);
  }
  // block merge: total count and mean first, then M2 about the block mean
  const CT bcnt = block_sum<CT>(cnt, lds);
  const CT bsum = block_sum<CT>(mean * cnt, lds);
  const CT bmean = bcnt > 0 ? bsum / bcnt : CT(0);
  const CT d = mean - bmean;
  const CT bm2 = block_sum<CT>(m2 + d * d * cnt, lds);
  if (threadIdx.x == 0) {
    CT* o = part + (c * s.splits + split) * 3;
    o[0] = bcnt; o[1] = bmean; o[2] = bm2;
  }
}

// One thread per channel: merge the slices; write the saved mean / inverse standard deviation, update the
// running statistics (the running variance takes the unbiased estimate, as cuDNN does), and leave
// coef[c] = scale * invstd, coef[C + c] = mean, coef[2 C + c] = bias for the element-wise pass.
template <typename PT, typename CT>
__global__ __launch_bounds__(256)
void bn_finalize_kernel(const CT* __restrict__ part, int64_t C, int splits, const PT* __restrict__ scale,
                        const PT* __restrict__ bias, double momentum, double eps, PT* running_mean,
                        PT* running_var, PT* save_mean, PT* save_invstd, CT* __restrict__ coef) {
  const int64_t c = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (c >= C) return;
  CT cnt = 0, mean = 0, m2 = 0;
  for (int k = 0; k < splits; ++k) {
    const CT* p = part + (c * splits + k) * 3;
    const CT nb = p[0];
    if (nb <= 0) continue;
    const CT n = cnt + nb;
    const CT delta = p[1] - mean;
    mean += delta * (nb / n);
    m2 += p[2] + delta * delta * (cnt * nb / n);
    cnt = n;
  }
  const CT var = cnt > 0 ? m2 / cnt : CT(0);
  CT invstd;
  if constexpr (std::is_same<CT, double>::value) invstd = 1.0 / sqrt(var + eps);
  else invstd = 1.0f / sqrtf(var + float(eps));
  if (save_mean) save_mean[c] = PT(mean);
  if (save_invstd) save_invstd[c] = PT(invstd);
  if (running_mean) running_mean[c] = PT((1.0 - momentum) * double(running_mean[c]) + momentum * double(mean));
  if (running_var) {
    const double unbiased = cnt > 1 ? double(m2) / (double(cnt) - 1.0) : double(var);
    running_var[c] = PT((1.0 - momentum) * double(running_var[c]) + momentum * unbiased);
  }
  coef[c] = CT(scale[c]) * invstd;
  coef[C + c] = mean;
  coef[2 * C + c] = CT(bias[c]);
}

// One load of V elements as it comes from memory; unpacked only after every load of the thread is issued.
template <typename T, int V>
struct BnRaw {
  u32x4 vec;
  T one;
  __device__ __forceinline__ void load(const T* p) {
    if constexpr (V == 1) one = *p;
    else vec = ld16(p);
  }
  template <typename CT>
  __device__ __forceinline__ void unpack(CT* f) const {
    if constexpr (V == 1) {
      f[0] = CT(Cvt<T>::load(&one));
    } else {
      float t[V];
      VecIO<T>::unpack(vec, t);
#pragma unroll
      for (int j = 0; j < V; ++j) f[j] = t[j];
    }
  }
};

// Channel of load v of a dense [N, C, H*W] array, and whether the whole wavefront shares it (it does unless the
// wavefront crosses from one plane into the next): then the channel's coefficients are fetched once per
// wavefront through the scalar unit instead of once per lane.
template <typename IT>
__device__ __forceinline__ IT bn_channel(IT v, IT hw_vec, IT C, bool& uniform) {
  const IT plane = v / hw_vec;
  const IT plane0 = IT(__builtin_amdgcn_readfirstlane(uint32_t(plane)));
  uniform = __builtin_amdgcn_ballot_w64(plane != plane0) == 0;
  return uniform ? plane0 % C : plane % C;
}

// y = (x - mean) * (scale * invstd) + bias; the mean is subtracted first: folding it into the constant term
// would cancel badly for a channel whose mean is large against its spread.  IT: index type (32-bit when the
// array allows it: the per-lane division is then a few instructions).
template <typename T, int V, typename CT, typename IT>
__global__ __launch_bounds__(256)
void bn_apply_kernel(const T* x, T* y, const CT* __restrict__ coef, IT total_loads, IT hw_vec, IT C) {
  const IT v = IT(blockIdx.x) * kStreamThreads + threadIdx.x;
  if (v >= total_loads) return;
  BnRaw<T, V> rx;
  rx.load(x + size_t(v) * V);
  bool uniform;
  const IT c = bn_channel<IT>(v, hw_vec, C, uniform);
  CT a, mean, b;
  if (uniform) {
    const IT c0 = IT(__builtin_amdgcn_readfirstlane(uint32_t(c)));
    a = coef[c0]; mean = coef[size_t(C) + c0]; b = coef[2 * size_t(C) + c0];
  } else {
    a = coef[c]; mean = coef[size_t(C) + c]; b = coef[2 * size_t(C) + c];
  }
  CT f[V];
  rx.unpack(f);
#pragma unroll
  for (int j = 0; j < V; ++j) f[j] = (f[j] - mean) * a + b;
  bn_store<T, V, CT>(y + size_t(v) * V, f);
}

// per-channel partial sums of dy and dy * (x - mean) * invstd -> part[(c * splits + split) * 2 ..]
template <typename T, int V, typename PT, typename CT>
__global__ __launch_bounds__(256)
void bn_bwd_stats_kernel(const T* __restrict__ dy, const T* __restrict__ x, BnShape s,
                         const PT* __restrict__ save_mean, const PT* __restrict__ save_invstd,
                         CT* __restrict__ part) {
  __shared__ CT lds[256];
  const int64_t c = blockIdx.x;
  const int split = blockIdx.y;
  const CT mean = CT(save_mean[c]), invstd = CT(save_invstd[c]);
  CT sdy = 0, sdyx = 0;
  for (BnWalk w(s, c, int64_t(split) * 256 + threadIdx.x, int64_t(s.splits) * 256, V); w.left > 0; w.next()) {
    CT g[V], f[V];
    bn_load<T, V, CT>(dy + w.off, g);
    bn_load<T, V, CT>(x + w.off, f);
#pragma unroll
    for (int j = 0; j < V; ++j) { sdy += g[j]; sdyx += g[j] * ((f[j] - mean) * invstd); }
  }
  sdy = block_sum<CT>(sdy, lds);
  sdyx = block_sum<CT>(sdyx, lds);
  if (threadIdx.x == 0) {
    CT* o = part + (c * s.splits + split) * 2;
    o[0] = sdy; o[1] = sdyx;
  }
}

// dscale = sum dy * xhat, dbias = sum dy; coefficients of dx = k0 * dy + k1 * (x - mean) + k2 with
//   dx = scale * invstd * (dy - dbias / m - xhat * dscale / m),  xhat = (x - mean) * invstd
template <typename PT, typename CT>
__global__ __launch_bounds__(256)
void bn_bwd_finalize_kernel(const CT* __restrict__ part, int64_t C, int splits, CT count,
                            const PT* __restrict__ scale, const PT* __restrict__ save_mean,
                            const PT* __restrict__ save_invstd, PT* dscale, PT* dbias, CT* __restrict__ coef) {
  const int64_t c = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (c >= C) return;
  CT sdy = 0, sdyx = 0;
  for (int k = 0; k < splits; ++k) {
    sdy += part[(c * splits + k) * 2];
    sdyx += part[(c * splits + k) * 2 + 1];
  }
  if (dscale) dscale[c] = PT(sdyx);
  if (dbias) dbias[c] = PT(sdy);
  const CT mean = CT(save_mean[c]), invstd = CT(save_invstd[c]);
  const CT a = CT(scale[c]) * invstd;
  coef[c] = a;
  coef[C + c] = -a * invstd * sdyx / count;
  coef[2 * C + c] = -a * sdy / count;
  coef[3 * C + c] = mean;
}

template <typename T, int V, typename CT, typename IT>
__global__ __launch_bounds__(256)
void bn_bwd_apply_kernel(const T* dy, const T* x, T* dx, const CT* __restrict__ coef, IT total_loads, IT hw_vec,
                         IT C) {
  const IT v = IT(blockIdx.x) * kStreamThreads + threadIdx.x;
  if (v >= total_loads) return;
  BnRaw<T, V> rg, rx;
  rg.load(dy + size_t(v) * V);
  rx.load(x + size_t(v) * V);
  bool uniform;
  const IT c = bn_channel<IT>(v, hw_vec, C, uniform);
  CT k0, k1, k2, mean;
  if (uniform) {
    const IT c0 = IT(__builtin_amdgcn_readfirstlane(uint32_t(c)));
    k0 = coef[c0]; k1 = coef[size_t(C) + c0]; k2 = coef[2 * size_t(C) + c0]; mean = coef[3 * size_t(C) + c0];
  } else {
    k0 = coef[c]; k1 = coef[size_t(C) + c]; k2 = coef[2 * size_t(C) + c]; mean = coef[3 * size_t(C) + c];
  }
  CT g[V], f[V];
  rg.unpack(g);
  rx.unpack(f);
#pragma unroll
  for (int j = 0; j < V; ++j) g[j] = k0 * g[j] + (k1 * (f[j] - mean) + k2);
  bn_store<T, V, CT>(dx + size_t(v) * V, g);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static int bn_splits(int64_t C, int64_t per_channel) {
  // enough workgroups to fill the chip (about 8 per compute unit), each with at least 8 loads per thread
  if (C <= 0) return 1;   // an empty array: callers return before launching anything
  const int64_t want = (int64_t(device_cu_count()) * 8 + C - 1) / C;
  const int64_t most = std::max<int64_t>(1, per_channel / (256 * 8));
  return int(std::max<int64_t>(1, std::min<int64_t>(std::min(want, most), 1024)));
}

template <int V>
static BnShape bn_shape(int64_t N, int64_t C, int64_t HW) {
  BnShape s{};
  s.N = N; s.C = C; s.HW = HW;
  s.hw_vec = HW / V;
  s.per_channel = N * s.hw_vec;
  s.splits = bn_splits(C, s.per_channel);
  return s;
}

static size_t bn_ws_bytes(int64_t N, int64_t C, int64_t HW, size_t ct_size) {
  // partials for the scalar decomposition (the larger one) + four coefficient rows
  const BnShape s = bn_shape<1>(N, C, HW);
  return (size_t(C) * size_t(s.splits) * 3 + size_t(C) * 4) * ct_size;
}

template <typename T, typename PT>
static int bn_fwd_typed(const void* x, const void* scale, const void* bias, void* y, double momentum, double eps,
                        void* running_mean, void* running_var, void* save_mean, void* save_invstd, int64_t N,
                        int64_t C, int64_t HW, void* ws, hipStream_t st) {
  using CT = typename BnCT<T>::type;
  CT* part = static_cast<CT*>(ws);
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  bool vec = false;
  if constexpr (!std::is_same<T, double>::value) {
    vec = HW % VecIO<T>::N == 0 && aligned16(x) && aligned16(y);
  }
  auto run = [&](auto vtag) -> int {
    constexpr int V = decltype(vtag)::value;
    const BnShape s = bn_shape<V>(N, C, HW);
    CT* coef = part + size_t(C) * size_t(s.splits) * 3;
    HK_REQUIRE(C <= 0x7fffffffLL && (N * C * s.hw_vec + kStreamThreads - 1) / kStreamThreads <= 0x7fffffffLL, HK_ERR_INVALID,
               "hk_batch_norm_fwd: array too large");
    HK_LAUNCH((bn_stats_kernel<T, V, CT>), dim3(unsigned(C), unsigned(s.splits)), dim3(256), 0, st, xp, s, part);
    int rc = launch_check("bn_stats_kernel");
    if (rc != HK_OK) return rc;
    HK_LAUNCH((bn_finalize_kernel<PT, CT>), dim3(unsigned((C + 255) / 256)), dim3(256), 0, st, part, C,
                       s.splits, static_cast<const PT*>(scale), static_cast<const PT*>(bias), momentum, eps,
                       static_cast<PT*>(running_mean), static_cast<PT*>(running_var), static_cast<PT*>(save_mean),
                       static_cast<PT*>(save_invstd), coef);
    rc = launch_check("bn_finalize_kernel");
    if (rc != HK_OK) return rc;
    const int64_t loads = N * C * s.hw_vec;
    profile_before(st);
    if (loads < 0x7fffffffLL) {
      HK_LAUNCH((bn_apply_kernel<T, V, CT, uint32_t>), dim3(unsigned((loads + kStreamThreads - 1) / kStreamThreads)), dim3(kStreamThreads), 0, st,
                         xp, yp, coef, uint32_t(loads), uint32_t(s.hw_vec), uint32_t(C));
    } else {
      HK_LAUNCH((bn_apply_kernel<T, V, CT, int64_t>), dim3(unsigned((loads + kStreamThreads - 1) / kStreamThreads)), dim3(kStreamThreads), 0, st,
                         xp, yp, coef, loads, s.hw_vec, C);
    }
    profile_after(st);
    return launch_check("bn_apply_kernel");
  };
  if constexpr (!std::is_same<T, double>::value) {
    if (vec) return run(std::integral_constant<int, VecIO<T>::N>{});
  }
  return run(std::integral_constant<int, 1>{});
}

template <typename T, typename PT>
static int bn_bwd_typed(const void* dy, const void* x, const void* scale, void* dx, void* dscale, void* dbias,
                        const void* save_mean, const void* save_invstd, int64_t N, int64_t C, int64_t HW, void* ws,
                        hipStream_t st) {
  using CT = typename BnCT<T>::type;
  CT* part = static_cast<CT*>(ws);
  bool vec = false;
  if constexpr (!std::is_same<T, double>::value) {
    vec = HW % VecIO<T>::N == 0 && aligned16(x) && aligned16(dy) && aligned16(dx);
  }
  auto run = [&](auto vtag) -> int {
    constexpr int V = decltype(vtag)::value;
    const BnShape s = bn_shape<V>(N, C, HW);
    CT* coef = part + size_t(C) * size_t(s.splits) * 3;
    HK_REQUIRE(C <= 0x7fffffffLL && (N * C * s.hw_vec + kStreamThreads - 1) / kStreamThreads <= 0x7fffffffLL, HK_ERR_INVALID,
               "hk_batch_norm_bwd: array too large");
    HK_LAUNCH((bn_bwd_stats_kernel<T, V, PT, CT>), dim3(unsigned(C), unsigned(s.splits)), dim3(256), 0, st,
                       static_cast<const T*>(dy), static_cast<const T*>(x), s, static_cast<const PT*>(save_mean),
                       static_cast<const PT*>(save_invstd), part);
    int rc = launch_check("bn_bwd_stats_kernel");
    if (rc != HK_OK) return rc;
    HK_LAUNCH((bn_bwd_finalize_kernel<PT, CT>), dim3(unsigned((C + 255) / 256)), dim3(256), 0, st, part, C,
                       s.splits, CT(N * HW), static_cast<const PT*>(scale), static_cast<const PT*>(save_mean),
                       static_cast<const PT*>(save_invstd), static_cast<PT*>(dscale), static_cast<PT*>(dbias), coef);
    rc = launch_check("bn_bwd_finalize_kernel");
    if (rc != HK_OK) return rc;
    const int64_t loads = N * C * s.hw_vec;
    profile_before(st);
    if (loads < 0x7fffffffLL) {
      HK_LAUNCH((bn_bwd_apply_kernel<T, V, CT, uint32_t>), dim3(unsigned((loads + kStreamThreads - 1) / kStreamThreads)), dim3(kStreamThreads), 0,
                         st, static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<T*>(dx), coef,
                         uint32_t(loads), uint32_t(s.hw_vec), uint32_t(C));
    } else {
      HK_LAUNCH((bn_bwd_apply_kernel<T, V, CT, int64_t>), dim3(unsigned((loads + kStreamThreads - 1) / kStreamThreads)), dim3(kStreamThreads), 0,
                         st, static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<T*>(dx), coef, loads,
                         s.hw_vec, C);
    }
    profile_after(st);
    return launch_check("bn_bwd_apply_kernel");
  };
  if constexpr (!std::is_same<T, double>::value) {
    if (vec) return run(std::integral_constant<int, VecIO<T>::N>{});
  }
  return run(std::integral_constant<int, 1>{});
}

static int bn_check(const char* who, int dtype, int64_t N, int64_t C, int64_t HW, const void* ws, size_t ws_bytes,
                    size_t* need) {
  HK_REQUIRE(N >= 0 && C >= 0 && HW >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  HK_REQUIRE(dtype == HK_FLOAT32 || dtype == HK_BFLOAT16 || dtype == HK_FLOAT16 || dtype == HK_FLOAT64,
             HK_ERR_UNSUPPORTED, "%s: not implemented for dtype %d", who, dtype);
  *need = 0;
  if (N * C * HW == 0) return HK_OK;   // before the split plan, which divides by C
  *need = bn_ws_bytes(N, C, HW, dtype == HK_FLOAT64 ? 8 : 4);
  HK_REQUIRE(ws != nullptr && ws_bytes >= *need, HK_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given",
             who, *need, ws_bytes);
  HK_REQUIRE(aligned16(ws), HK_ERR_INVALID, "%s: workspace must be 16-byte aligned", who);
  return HK_OK;
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_batch_norm_workspace_bytes(int dtype, int64_t N, int64_t C, int64_t HW, size_t* bytes) {
  HK_REQUIRE(bytes, HK_ERR_INVALID, "hk_batch_norm_workspace_bytes: null output");
  HK_REQUIRE(N >= 0 && C >= 0 && HW >= 0, HK_ERR_INVALID, "hk_batch_norm_workspace_bytes: negative shape");
  *bytes = (N * C * HW == 0) ? 0 : bn_ws_bytes(N, C, HW, dtype == HK_FLOAT64 ? 8 : 4);
  return HK_OK;
}

int hk_batch_norm_fwd(int dtype, const void* x, const void* scale, const void* bias, void* y, double momentum,
                      double eps, void* running_mean, void* running_var, void* save_mean, void* save_invstd,
                      int64_t N, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                      hkStream_t stream) {
  size_t need = 0;
  int rc = bn_check("hk_batch_norm_fwd", dtype, N, C, HW, workspace, workspace_bytes, &need);
  if (rc != HK_OK) return rc;
  if (N * C * HW == 0) return HK_OK;
  HK_REQUIRE(x && scale && bias && y, HK_ERR_INVALID, "hk_batch_norm_fwd: null input/output");
  hipStream_t st = as_hip(stream);
  switch (dtype) {
    case HK_FLOAT32:
      return bn_fwd_typed<float, float>(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean,
                                        save_invstd, N, C, HW, workspace, st);
    case HK_BFLOAT16:
      return bn_fwd_typed<bf16, float>(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean,
                                       save_invstd, N, C, HW, workspace, st);
    case HK_FLOAT16:
      return bn_fwd_typed<fp16, float>(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean,
                                       save_invstd, N, C, HW, workspace, st);
    default:
      return bn_fwd_typed<double, double>(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean,
                                          save_invstd, N, C, HW, workspace, st);
  }
}

int hk_batch_norm_bwd(int dtype, const void* dy, const void* x, const void* scale, void* dx, void* dscale,
                      void* dbias, const void* save_mean, const void* save_invstd, int64_t N, int64_t C,
                      int64_t HW, void* workspace, size_t workspace_bytes, hkStream_t stream) {
  size_t need = 0;
  int rc = bn_check("hk_batch_norm_bwd", dtype, N, C, HW, workspace, workspace_bytes, &need);
  if (rc != HK_OK) return rc;
  if (N * C * HW == 0) return HK_OK;
  HK_REQUIRE(dy && x && scale && dx && save_mean && save_invstd, HK_ERR_INVALID,
             "hk_batch_norm_bwd: null input/output");
  hipStream_t st = as_hip(stream);
  switch (dtype) {
    case HK_FLOAT32:
      return bn_bwd_typed<float, float>(dy, x, scale, dx, dscale, dbias, save_mean, save_invstd, N, C, HW, workspace, st);
    case HK_BFLOAT16:
      return bn_bwd_typed<bf16, float>(dy, x, scale, dx, dscale, dbias, save_mean, save_invstd, N, C, HW, workspace, st);
    case HK_FLOAT16:
      return bn_bwd_typed<fp16, float>(dy, x, scale, dx, dscale, dbias, save_mean, save_invstd, N, C, HW, workspace, st);
    default:
      return bn_bwd_typed<double, double>(dy, x, scale, dx, dscale, dbias, save_mean, save_invstd, N, C, HW, workspace, st);
  }
}

} // extern "C"
