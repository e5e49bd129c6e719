// LayerNorm / RMSNorm forward and backward for gfx950.
//
// Forward: a row lives in registers as packed 128-bit vectors (one HBM read),
// statistics are Welford moments merged with Chan's update across lanes (DPP,
// equal-count form when the row fills every lane) and waves (LDS), output is
// written with 128-bit stores.  One wavefront per
// row for short rows, one workgroup per row for long rows.
//
// Backward: a persistent grid walks the rows; every thread owns a fixed set of
// columns, keeps the dgamma / dbeta column sums of its rows in registers, and the
// workgroup writes ONE fp32 partial row per block which a small second kernel
// folds into dgamma / dbeta.
#include "hk_common.cuh"

#include <algorithm>
#include <mutex>
#include <type_traits>

namespace hk {

// ===========================================================================
// forward
// ===========================================================================
struct NormFwdArgs {
  const void* x;
  const void* residual;
  const void* gamma;
  const void* beta;
  void* y;
  void* x_out;
  void* mean;
  void* stat;
  int64_t rows;
  int cols;
  int nvec;
  float eps;
  float inv_cols;
  int is_rms;
  int stat_kind;
  int stats_f32;
  int stream_store;
};

template <typename T>
__device__ __forceinline__ void store_stat(void* base, int64_t row, float v, int stats_f32) {
  if (base == nullptr) return;
  if (stats_f32) static_cast<float*>(base)[row] = v;
  else Cvt<T>::store(static_cast<T*>(base) + row, v);
}

template <typename T>
__device__ __forceinline__ float load_stat(const void* base, int64_t row, int stats_f32) {
  if (stats_f32) return static_cast<const float*>(base)[row];
  return Cvt<T>::load(static_cast<const T*>(base) + row);
}

// T: element type; NV: 16-byte vectors per thread; WAVE_ROW: one wavefront per
// row (4 rows per 256-thread block) instead of one workgroup per row;
// HAS_RES: x = x0 + residual is formed in fp32 and optionally written back.
template <typename T, int NV, bool WAVE_ROW, bool HAS_RES>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024)
void norm_fwd_kernel(NormFwdArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves * 3];

  const int tpr = WAVE_ROW ? kWave : int(blockDim.x);
  const int t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  const int64_t row = WAVE_ROW
      ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index()
      : int64_t(blockIdx.x);
  if (WAVE_ROW && row >= a.rows) return;  // wave-uniform; no block barrier in this mode
  const int nwaves = WAVE_ROW ? 1 : int(blockDim.x >> 6);

  const T* xr = static_cast<const T*>(a.x) + row * int64_t(a.cols);
  u32x4 raw[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) raw[i] = u32x4{0, 0, 0, 0};
  [[maybe_unused]] float xf[HAS_RES ? NV * VEC : 1];

#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if (v < a.nvec) raw[i] = ld16(xr + v * VEC);
  }
  if constexpr (HAS_RES) {
    const T* rr = static_cast<const T*>(a.residual) + row * int64_t(a.cols);
    T* xo = a.x_out ? static_cast<T*>(a.x_out) + row * int64_t(a.cols) : nullptr;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * tpr + t;
      if (v < a.nvec) {
        float f0[VEC], f1[VEC];
        VecIO<T>::unpack(raw[i], f0);
        VecIO<T>::unpack(ld16(rr + v * VEC), f1);
#pragma unroll
        for (int j = 0; j < VEC; ++j) xf[i * VEC + j] = f0[j] + f1[j];
        if (xo) st16(xo + v * VEC, VecIO<T>::pack(&xf[i * VEC]));
      }
    }
  }

  auto get = [&](int i, float* f) {
    if constexpr (HAS_RES) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) f[j] = xf[i * VEC + j];
    } else {
      VecIO<T>::unpack(raw[i], f);
    }
  };

  float mu, rs, var;
  if (a.is_rms) {
    SumTuple<2> s;
    s.v[0] = 0.f; s.v[1] = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i * tpr + t < a.nvec) {
        float f[VEC];
        get(i, f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) { s.v[0] += f[j]; s.v[1] = fmaf(f[j], f[j], s.v[1]); }
      }
    }
    s = WAVE_ROW ? wave_allreduce_tuple(s) : group_allreduce_tuple(s, red, 0, nwaves);
    mu = s.v[0] * a.inv_cols;
    const float ms = s.v[1] * a.inv_cols;  // mean(x^2) = var + mu^2
    var = fmaxf(ms - mu * mu, 0.f);
    rs = 1.0f / sqrtf(ms + a.eps);
  } else {
    // Welford statistics, merged with Chan's parallel update: each thread forms (count, mean, M2) of the
    // elements it holds in registers, lanes merge through a DPP butterfly, waves through LDS.  When every
    // thread holds the same count (the row fills all vector slots: a uniform test) each butterfly step
    // merges equal-sized halves and needs no reciprocal; a ragged row takes the general update.
    float s = 0.f;
    int cnt = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i * tpr + t < a.nvec) {
        float f[VEC];
        get(i, f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) s += f[j];
        cnt += VEC;
      }
    }
    const bool even = a.nvec == NV * tpr;                    // uniform
    const float mean_t = even ? s * (1.0f / float(NV * VEC)) : (cnt > 0 ? s / float(cnt) : 0.f);
    float m2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (i * tpr + t < a.nvec) {
        float f[VEC];
        get(i, f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) { const float d = f[j] - mean_t; m2 = fmaf(d, d, m2); }
      }
    }
    MomentTuple m;
    m.v[0] = float(cnt); m.v[1] = mean_t; m.v[2] = m2;
    if (even) {
      EqualMomentTuple e;
      e.v[0] = m.v[0]; e.v[1] = m.v[1]; e.v[2] = m.v[2];
      e = wave_allreduce_tuple(e);
      m.v[0] = e.v[0]; m.v[1] = e.v[1]; m.v[2] = e.v[2];
    } else {
      m = wave_allreduce_tuple(m);
    }
    // waves are merged one after the other (growing count on one side): the general update
    if (!WAVE_ROW) m = group_combine_tuple(m, red, 0, nwaves);
    mu = m.v[1];
    var = m.v[2] * a.inv_cols;
    rs = 1.0f / sqrtf(var + a.eps);
  }

  if (t == 0) {
    store_stat<T>(a.mean, row, mu, a.stats_f32);
    store_stat<T>(a.stat, row, a.stat_kind == HK_STAT_VAR ? var : rs, a.stats_f32);
  }

  const float shift = a.is_rms ? 0.f : mu;
  T* yr = static_cast<T*>(a.y) + row * int64_t(a.cols);
  // gamma / beta are fetched here, after the reduction: holding them in registers across it was measured
  // slower (fewer resident waves) than these cache hits.  All of them are issued before the first is
  // unpacked: a load inside the per-vector branch on the pointer would wait for the one before it.
  const T* gp = static_cast<const T*>(a.gamma);
  const T* bp = static_cast<const T*>(a.beta);
  u32x4 rawg[NV], rawb[NV];
  if (gp) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * tpr + t;
      rawg[i] = u32x4{0, 0, 0, 0};
      if (v < a.nvec) rawg[i] = ld16_keep(gp + v * VEC);
    }
  }
  if (bp) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * tpr + t;
      rawb[i] = u32x4{0, 0, 0, 0};
      if (v < a.nvec) rawb[i] = ld16_keep(bp + v * VEC);
    }
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if (v < a.nvec) {
      float f[VEC], g[VEC], b[VEC];
      get(i, f);
      if (gp) VecIO<T>::unpack(rawg[i], g);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) g[j] = 1.f;
      }
      if (bp) VecIO<T>::unpack(rawb[i], b);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) b[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) f[j] = fmaf(g[j], rs * (f[j] - shift), b[j]);
      const u32x4 o = VecIO<T>::pack(f);
      if (a.stream_store) st16_stream(yr + v * VEC, o);
      else st16(yr + v * VEC, o);
    }
  }
}

// Fallback for rows that are not a whole number of 16-byte vectors, are not
// 16-byte aligned, or do not fit the register file: one workgroup per row,
// three strided passes (the re-reads hit L2).  CT is the arithmetic type.
template <typename CT>
__device__ __forceinline__ CT block_sum_generic(CT v, CT* lds) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
    if (tid < s) lds[tid] += lds[tid + s];
    __syncthreads();
  }
  CT r = lds[0];
  __syncthreads();
  return r;
}

template <typename T, typename CT>
struct GenericIO {
  static __device__ __forceinline__ CT ld(const T* p) { return CT(Cvt<T>::load(p)); }
  static __device__ __forceinline__ void st(T* p, CT v) { Cvt<T>::store(p, v); }
};

template <typename T, typename CT>
__global__ __launch_bounds__(256)
void norm_fwd_generic_kernel(NormFwdArgs a) {
  __shared__ CT lds[256];
  const int64_t row = blockIdx.x;
  const T* xr = static_cast<const T*>(a.x) + row * int64_t(a.cols);
  const T* rr = a.residual ? static_cast<const T*>(a.residual) + row * int64_t(a.cols) : nullptr;
  T* xo = a.x_out ? static_cast<T*>(a.x_out) + row * int64_t(a.cols) : nullptr;
  auto ldx = [&](int c) -> CT {
    CT v = GenericIO<T, CT>::ld(xr + c);
    if (rr) v += GenericIO<T, CT>::ld(rr + c);
    return v;
  };
  CT s = 0, ss = 0;
  for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
    const CT v = ldx(c);
    if (xo) GenericIO<T, CT>::st(xo + c, v);
    s += v;
    ss += v * v;
  }
  s = block_sum_generic<CT>(s, lds);
  const CT inv = CT(1) / CT(a.cols);
  const CT mu = s * inv;
  CT var, rs;
  if (a.is_rms) {
    ss = block_sum_generic<CT>(ss, lds);
    const CT ms = ss * inv;
    var = ms - mu * mu;
    if (var < CT(0)) var = CT(0);
    rs = CT(1) / sqrt(ms + CT(a.eps));
  } else {
    CT m2 = 0;
    for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
      const CT d = ldx(c) - mu;
      m2 += d * d;
    }
    m2 = block_sum_generic<CT>(m2, lds);
    var = m2 * inv;
    rs = CT(1) / sqrt(var + CT(a.eps));
  }
  if (threadIdx.x == 0) {
    const CT st = a.stat_kind == HK_STAT_VAR ? var : rs;
    if (a.mean) {
      if (a.stats_f32) static_cast<float*>(a.mean)[row] = float(mu);
      else GenericIO<T, CT>::st(static_cast<T*>(a.mean) + row, mu);
    }
    if (a.stat) {
      if (a.stats_f32) static_cast<float*>(a.stat)[row] = float(st);
      else GenericIO<T, CT>::st(static_cast<T*>(a.stat) + row, st);
    }
  }
  const CT shift = a.is_rms ? CT(0) : mu;
  T* yr = static_cast<T*>(a.y) + row * int64_t(a.cols);
  const T* gp = static_cast<const T*>(a.gamma);
  const T* bp = static_cast<const T*>(a.beta);
  for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
    const CT g = gp ? GenericIO<T, CT>::ld(gp + c) : CT(1);
    const CT b = bp ? GenericIO<T, CT>::ld(bp + c) : CT(0);
    GenericIO<T, CT>::st(yr + c, g * (rs * (ldx(c) - shift)) + b);
  }
}

static inline int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <typename T, bool WAVE_ROW, bool HAS_RES>
static int launch_norm_fwd_nv(const NormFwdArgs& a, int nv, dim3 grid, dim3 block, hipStream_t s) {
  profile_before(s);
  switch (nv) {
    case 1: hipLaunchKernelGGL((norm_fwd_kernel<T, 1, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 2: hipLaunchKernelGGL((norm_fwd_kernel<T, 2, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 3: hipLaunchKernelGGL((norm_fwd_kernel<T, 3, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 4: hipLaunchKernelGGL((norm_fwd_kernel<T, 4, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 5: hipLaunchKernelGGL((norm_fwd_kernel<T, 5, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 6: hipLaunchKernelGGL((norm_fwd_kernel<T, 6, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 8: hipLaunchKernelGGL((norm_fwd_kernel<T, 8, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    case 16: hipLaunchKernelGGL((norm_fwd_kernel<T, 16, WAVE_ROW, HAS_RES>), grid, block, 0, s, a); break;
    default:
      set_last_error("norm_fwd: no kernel for %d vectors per thread", nv);
      return HK_ERR_UNSUPPORTED;
  }
  profile_after(s);
  return launch_check("norm_fwd_kernel");
}

// Picks threads-per-row and vectors-per-thread for a row of `nvec` 16-byte
// vectors.  Returns false when the row does not fit the register kernels.
static bool pick_row_shape(int nvec, int forced_threads, int max_nv, int wave_row_max_nv,
                           int* threads, int* nv) {
  if (forced_threads > 0) {
    int t = std::min(1024, std::max(64, (forced_threads + 63) / 64 * 64));
    int n = pow2_ceil((nvec + t - 1) / t);
    if (n > max_nv) return false;
    *threads = t;
    *nv = n;
    return true;
  }
  // short rows: one wavefront per row
  if (nvec <= 64 * wave_row_max_nv && nvec <= 256) {
    *threads = 64;
    *nv = pow2_ceil((nvec + 63) / 64);
    return true;
  }
  // medium rows (measured on MI355X: 4096 / 5120 bf16 columns, 4096 fp32
  // columns): small workgroups of 128..256 threads per row stream fastest.
  // First choice: the fewest vectors per thread that fill every lane exactly
  // (5120 bf16 columns = 640 vectors = 128 threads x 5): no idle lanes, and the
  // statistics merge takes its equal-count form.
  static const int kCounts[] = {2, 3, 4, 5, 6, 8};
  for (int n : kCounts) {
    if (n > max_nv) break;
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 256 && n * t == nvec) {
      *threads = t;
      *nv = n;
      return true;
    }
  }
  for (int n = 2; n <= max_nv; n <<= 1) {
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 256) {
      *threads = t;
      *nv = n;
      return true;
    }
  }
  // long rows: one workgroup per row, smallest power-of-two vector count that
  // keeps the block within 1024 threads
  for (int n = 4; n <= max_nv; n <<= 1) {
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 1024) {
      *threads = t;
      *nv = n;
      return true;
    }
  }
  return false;
}

template <typename T>
static int norm_fwd_typed(NormFwdArgs a, hipStream_t s) {
  constexpr int VEC = VecIO<T>::N;
  const bool vec_ok = (a.cols % VEC == 0) && aligned16(a.x) && aligned16(a.y) &&
                      aligned16(a.gamma) && aligned16(a.beta) && aligned16(a.residual) &&
                      aligned16(a.x_out);
  int threads = 0, nv = 0;
  a.nvec = a.cols / VEC;
  const bool has_res = a.residual != nullptr;
  // with a residual the summed row is kept unpacked: halve the budget
  const int max_nv = has_res ? (VEC == 4 ? 16 : 8) : 16;
  const int wave_nv = has_res ? (VEC == 4 ? 8 : 4) : (VEC == 4 ? 16 : 8);
  if (vec_ok && pick_row_shape(a.nvec, tune_get(TUNE_NORM_FWD_THREADS), max_nv, wave_nv, &threads, &nv)) {
    if (threads == 64) {
      dim3 grid(unsigned((a.rows + 3) / 4)), block(256);
      return has_res ? launch_norm_fwd_nv<T, true, true>(a, nv, grid, block, s)
                     : launch_norm_fwd_nv<T, true, false>(a, nv, grid, block, s);
    }
    dim3 grid{unsigned(a.rows)}, block{unsigned(threads)};
    return has_res ? launch_norm_fwd_nv<T, false, true>(a, nv, grid, block, s)
                   : launch_norm_fwd_nv<T, false, false>(a, nv, grid, block, s);
  }
  hipLaunchKernelGGL((norm_fwd_generic_kernel<T, float>), dim3(unsigned(a.rows)), dim3(256), 0, s, a);
  return launch_check("norm_fwd_generic_kernel");
}

static int norm_fwd_dispatch(int dtype, NormFwdArgs& a, hipStream_t s, const char* who) {
  HK_REQUIRE(a.rows >= 0 && a.cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  if (a.rows == 0 || a.cols == 0) return HK_OK;
  HK_REQUIRE(a.rows <= 0x7fffffffLL && a.cols <= 0x3fffffff, HK_ERR_INVALID,
             "%s: shape [%lld, %d] too large", who, (long long)a.rows, a.cols);
  HK_REQUIRE(a.x && a.y, HK_ERR_INVALID, "%s: null input/output", who);
  a.inv_cols = 1.0f / float(a.cols);
  const int st = tune_get(TUNE_STREAM_STORES);
  a.stream_store = (st == 2) ? 0 : 1;
  switch (dtype) {
    case HK_FLOAT32: return norm_fwd_typed<float>(a, s);
    case HK_BFLOAT16: return norm_fwd_typed<bf16>(a, s);
    case HK_FLOAT16: return norm_fwd_typed<fp16>(a, s);
    case HK_FLOAT64:
      hipLaunchKernelGGL((norm_fwd_generic_kernel<double, double>), dim3(unsigned(a.rows)), dim3(256), 0, s, a);
      return launch_check("norm_fwd_generic_kernel<double>");
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

// ===========================================================================
// backward
// ===========================================================================
enum NormBwdMode { BWD_LN = 0, BWD_RMS = 1, BWD_LN_MEMEFF = 2 };

struct NormBwdArgs {
  const void* dy;
  const void* x;        // forward input, or forward output in BWD_LN_MEMEFF
  const void* gamma;
  const void* beta;     // BWD_LN_MEMEFF only
  const void* mean;
  const void* stat;
  const void* dx_in;    // optional upstream gradient added to dx
  void* dx;
  void* dres;           // optional second copy of dx (dresidual)
  float* part_dgamma;   // [grid, cols]
  float* part_dbeta;    // [grid, cols]
  int64_t rows;
  int cols;
  int nvec;
  int tpr;              // threads per row (multiple of 64)
  float eps;
  float inv_cols;
  int stat_kind;
  int stats_f32;
  int clamp_gamma;
  int stream_store;
};

__device__ __forceinline__ float clamp_by_magnitude(float g, float eps) {
  // |g| < eps is pushed out to +-eps keeping the sign (zero counts as positive)
  if (g >= 0.f) return g < eps ? eps : g;
  return g > -eps ? -eps : g;
}

// Column-owner backward kernel.  A group of `tpr` threads walks rows; thread t
// owns the same columns in every row, so its dgamma / dbeta sums stay in
// registers.  With xc = x - mu (x for RMSNorm), t = dy * gamma and
// m2 = mean(t * xc):   dx = rs * t - rs * mean(t) - xc * rs^3 * m2,
// two fused multiply-adds per element once the row sums are known.
//
// PF rows per thread group are in flight at any time (a ring of register slots,
// refilled as soon as a slot has been unpacked).  The steady-state loop is
// written without a single branch around a memory instruction: out-of-range
// rows are clamped instead of skipped, EXACT says that no thread has a column
// past the row's end, STATS_F32 fixes the statistics' type.  Only then does the
// compiler count outstanding loads exactly; any branch in the loop makes it
// wait for all of them at every step, which flattens the ring to depth one.
// Rows that do not fill a whole round of PF steps go through the same step with
// its guards switched on.
template <typename T, int NV, int MODE, int PF, bool EXACT, bool STATS_F32>
__global__ __launch_bounds__(NV == 1 ? 1024 : 512)
void norm_bwd_kernel(NormBwdArgs a) {
  constexpr int VEC = VecIO<T>::N;
  constexpr int NE = NV * VEC;
  using StatT = typename std::conditional<STATS_F32, float, T>::type;
  extern __shared__ float lds[];           // [rows_per_block, cols] column-sum staging
  __shared__ float red[2][kMaxWaves * 2];  // double-buffered by step parity

  const int tpr = a.tpr;                   // multiple of 64: a wavefront never straddles two rows
  const int rpb = int(blockDim.x) / tpr;
  const int group = __builtin_amdgcn_readfirstlane(int(threadIdx.x) / tpr);
  const int t = int(threadIdx.x) - group * tpr;
  const int waves_per_group = tpr >> 6;
  const int first_wave = group * waves_per_group;

  // column vectors of this thread; a thread past the row's end (only when !EXACT) reads the last vector
  // again and has its dy forced to zero, so it adds nothing and stores nothing
  int vidx[NV];
  bool vin[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    vin[i] = EXACT || v < a.nvec;
    vidx[i] = vin[i] ? v : a.nvec - 1;
  }

  // gamma (and beta) of this thread's columns as fp32; a missing gamma is all ones
  float gm[NE];
  [[maybe_unused]] float bt[MODE == BWD_LN_MEMEFF ? NE : 1];
  {
    const T* gp = static_cast<const T*>(a.gamma);
    const T* bp = static_cast<const T*>(a.beta);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) gm[i * VEC + j] = 1.f;
      if (gp) VecIO<T>::unpack(ld16_keep(gp + vidx[i] * VEC), &gm[i * VEC]);
      if constexpr (MODE == BWD_LN_MEMEFF) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) bt[i * VEC + j] = 0.f;
        if (bp) VecIO<T>::unpack(ld16_keep(bp + vidx[i] * VEC), &bt[i * VEC]);
      }
    }
  }
  const bool clamp = a.clamp_gamma != 0 || MODE == BWD_LN_MEMEFF;

  float dg[NE], db[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) { dg[e] = 0.f; db[e] = 0.f; }

  const int64_t stride = int64_t(gridDim.x) * rpb;
  const int64_t last_row = a.rows - 1;
  u32x4 nx[PF][NV], ndy[PF][NV];
  StatT nmu[PF], nsv[PF];
  const StatT* meanp = static_cast<const StatT*>(a.mean);
  const StatT* statp = static_cast<const StatT*>(a.stat);
  // loads of row r into slot d; r past the end re-reads the last row (its results are never used)
  auto issue = [&](auto slot, int64_t r) {
    constexpr int d = decltype(slot)::value;
    const int64_t rc = r < last_row ? r : last_row;
    if constexpr (MODE == BWD_LN) nmu[d] = meanp[rc];
    nsv[d] = statp[rc];
    const T* xr = static_cast<const T*>(a.x) + rc * int64_t(a.cols);
    const T* dyr = static_cast<const T*>(a.dy) + rc * int64_t(a.cols);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      nx[d][i] = ld16(xr + vidx[i] * VEC);
      ndy[d][i] = ld16(dyr + vidx[i] * VEC);
    }
  };
  int64_t row0 = int64_t(blockIdx.x) * rpb + group;
  static_for<PF>([&](auto slot) { issue(slot, row0 + decltype(slot)::value * stride); });

  int parity = 0;
  // guarded: check that the slot's row exists (the tail); otherwise it is known to
  auto step = [&](auto slot, auto guarded) {
    constexpr int d = decltype(slot)::value;
    constexpr bool GUARD = decltype(guarded)::value;
    const int64_t row = row0 + d * stride;
    const bool valid = !GUARD || row < a.rows;
    float xs[NE], ts[NE];                 // xc (x_hat in the memory-efficient mode) and dy * gamma
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      VecIO<T>::unpack(nx[d][i], &xs[i * VEC]);
      VecIO<T>::unpack(ndy[d][i], &ts[i * VEC]);
      if (!EXACT) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) ts[i * VEC + j] = vin[i] ? ts[i * VEC + j] : 0.f;
      }
    }
    [[maybe_unused]] float mu = 0.f;
    if constexpr (MODE == BWD_LN) mu = Cvt<StatT>::to_float(nmu[d]);
    const float sv = Cvt<StatT>::to_float(nsv[d]);
    const float rs = a.stat_kind == HK_STAT_VAR ? 1.0f / sqrtf(sv + a.eps) : sv;
    // the slot is free again: refill it with the row PF steps ahead
    issue(slot, row + int64_t(PF) * stride);

    SumTuple<2> s;
    s.v[0] = 0.f; s.v[1] = 0.f;
    // new column sums go to copies first: a guarded step of a missing row must leave dg / db alone
    // without a branch around the arithmetic
    auto accumulate = [&](auto clamped) {
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const float dz = (GUARD && !valid) ? 0.f : ts[e];
        if constexpr (MODE == BWD_LN_MEMEFF) {
          const float yb = xs[e] - bt[e];
          const float kg = clamp_by_magnitude(gm[e], a.eps);
          const float xhat = yb / kg;
          s.v[0] = fmaf(dz, gm[e], s.v[0]);
          s.v[1] = fmaf(dz, yb, s.v[1]);
          dg[e] = fmaf(dz, xhat, dg[e]);
          db[e] += dz;
          xs[e] = xhat;
          ts[e] = dz * kg;
        } else {
          const float xc = (MODE == BWD_RMS) ? xs[e] : xs[e] - mu;
          const float dzr = dz * rs;
          const float q = dzr * gm[e];
          s.v[1] = fmaf(q, xc, s.v[1]);
          if (MODE != BWD_RMS) s.v[0] += q;
          dg[e] = fmaf(dzr, xc, dg[e]);
          db[e] += dz;
          xs[e] = xc;
          // the per-element term of dx uses the clamped gamma when asked to
          if constexpr (decltype(clamped)::value) ts[e] = dzr * clamp_by_magnitude(gm[e], a.eps);
          else ts[e] = q;
        }
      }
    };
    if (clamp) accumulate(std::true_type{});   // uniform
    else accumulate(std::false_type{});

    s = group_allreduce_tuple(s, red[parity], first_wave, waves_per_group);
    parity ^= 1;
    if (valid) {
      // plain modes: s0 = rs * sum(dy g), s1 = rs * sum(dy g xc);  dx = q - s0/n - xc * rs^2 * s1/n
      // memory-efficient: s0 = sum(dy g), s1 = sum(dy (y - beta));   dx = rs * (dy kg - s0/n - xhat * s1/n)
      float rc1, k3;
      if constexpr (MODE == BWD_LN_MEMEFF) {
        rc1 = rs * s.v[0] * a.inv_cols;
        k3 = rs * s.v[1] * a.inv_cols;
      } else {
        rc1 = (MODE == BWD_RMS) ? 0.f : s.v[0] * a.inv_cols;
        k3 = rs * rs * s.v[1] * a.inv_cols;
      }
      T* dxr = static_cast<T*>(a.dx) + row * int64_t(a.cols);
      T* drr = a.dres ? static_cast<T*>(a.dres) + row * int64_t(a.cols) : nullptr;
      const T* dir = a.dx_in ? static_cast<const T*>(a.dx_in) + row * int64_t(a.cols) : nullptr;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        if (EXACT || vin[i]) {
          const int v = vidx[i];
          float o[VEC];
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float base = (MODE == BWD_LN_MEMEFF) ? fmaf(ts[i * VEC + j], rs, -rc1)
                                                       : ts[i * VEC + j] - rc1;
            o[j] = fmaf(-xs[i * VEC + j], k3, base);
          }
          if (dir) {
            float u[VEC];
            VecIO<T>::unpack(ld16(dir + v * VEC), u);
#pragma unroll
            for (int j = 0; j < VEC; ++j) o[j] += u[j];
          }
          const u32x4 pk = VecIO<T>::pack(o);
          if (a.stream_store) st16_stream(dxr + v * VEC, pk);
          else st16(dxr + v * VEC, pk);
          if (drr) st16(drr + v * VEC, pk);
        }
      }
    }
  };
  // Every thread of the block takes the same number of steps (both loop bounds are block-uniform), so
  // the barrier inside the group reduction is reached by all of them.
  int64_t base = int64_t(blockIdx.x) * rpb;
  const int64_t round = int64_t(PF) * stride;
  // rounds in which every slot of every group of this block holds an existing row
#pragma nounroll
  for (; base + int64_t(PF - 1) * stride + rpb <= a.rows; base += round) {
    static_for<PF>([&](auto slot) { step(slot, std::false_type{}); });
    row0 += round;
  }
#pragma nounroll
  for (; base < a.rows; base += round) {
    static_for<PF>([&](auto slot) { step(slot, std::true_type{}); });
    row0 += round;
  }

  // fold the row groups of this block, then write one partial row per block
  float* outs[2] = {a.part_dgamma, a.part_dbeta};
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    if (outs[which] == nullptr) continue;
    float* acc = which == 0 ? dg : db;
    __syncthreads();
    if (rpb > 1) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = i * tpr + t;
        if (v < a.nvec) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) lds[group * a.cols + v * VEC + j] = acc[i * VEC + j];
        }
      }
      __syncthreads();
    }
    if (group == 0) {
      float* dst = outs[which] + int64_t(blockIdx.x) * a.cols;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = i * tpr + t;
        if (v < a.nvec) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            float r = acc[i * VEC + j];
            for (int g = 1; g < rpb; ++g) r += lds[g * a.cols + v * VEC + j];
            dst[v * VEC + j] = r;
          }
        }
      }
    }
  }
}

// Folds the [nparts, cols] fp32 partial rows into dgamma / dbeta of type T.
// blockIdx.y picks dgamma / dbeta; a block covers 128 columns as 32 float4
// column groups x 16 row slices, every slice keeps 8 independent loads in
// flight, slices are folded through LDS.
template <typename T>
__global__ __launch_bounds__(512)
void norm_bwd_finalize_kernel(const float* __restrict__ part_dgamma,
                              const float* __restrict__ part_dbeta, T* dgamma, T* dbeta,
                              int nparts, int cols) {
  constexpr int U = 8;
  __shared__ float lds[16][32][4];
  const float* part = blockIdx.y == 0 ? part_dgamma : part_dbeta;
  T* out = blockIdx.y == 0 ? dgamma : dbeta;
  if (part == nullptr || out == nullptr) return;     // uniform over the block
  const int cg = threadIdx.x & 31, slice = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + cg) * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {                                     // cols is a multiple of 4 on this path
    int r = slice;
    for (; r + (U - 1) * 16 < nparts; r += U * 16) {
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = ld16_keep(part + int64_t(r + u * 16) * cols + c);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        acc[0] += u2f(v[u].x); acc[1] += u2f(v[u].y); acc[2] += u2f(v[u].z); acc[3] += u2f(v[u].w);
      }
    }
    for (; r < nparts; r += 16) {
      const u32x4 v = ld16_keep(part + int64_t(r) * cols + c);
      acc[0] += u2f(v.x); acc[1] += u2f(v.y); acc[2] += u2f(v.z); acc[3] += u2f(v.w);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) lds[slice][cg][k] = acc[k];
  __syncthreads();
  if (threadIdx.x < 128) {
    const int g = threadIdx.x >> 2, k = threadIdx.x & 3;
    const int oc = (blockIdx.x * 32 + g) * 4 + k;
    float s = 0.f;
#pragma unroll
    for (int sl = 0; sl < 16; ++sl) s += lds[sl][g][k];
    if (oc < cols) Cvt<T>::store(out + oc, s);
  }
}

// Fallback backward for rows the register kernel cannot take: one workgroup
// per row for dx, then a column kernel for dgamma / dbeta (re-reads dy and x).
template <typename T, typename CT>
__global__ __launch_bounds__(256)
void norm_bwd_generic_dx_kernel(NormBwdArgs a, int mode) {
  __shared__ CT lds[256];
  const int64_t row = blockIdx.x;
  const T* xr = static_cast<const T*>(a.x) + row * int64_t(a.cols);
  const T* dyr = static_cast<const T*>(a.dy) + row * int64_t(a.cols);
  const T* gp = static_cast<const T*>(a.gamma);
  const T* bp = static_cast<const T*>(a.beta);
  CT mu = 0;
  if (mode == BWD_LN) {
    mu = a.stats_f32 ? CT(static_cast<const float*>(a.mean)[row])
                     : GenericIO<T, CT>::ld(static_cast<const T*>(a.mean) + row);
  }
  const CT sv = a.stats_f32 ? CT(static_cast<const float*>(a.stat)[row])
                            : GenericIO<T, CT>::ld(static_cast<const T*>(a.stat) + row);
  const CT rs = a.stat_kind == HK_STAT_VAR ? CT(1) / sqrt(sv + CT(a.eps)) : sv;
  const bool clamp = a.clamp_gamma != 0 || mode == BWD_LN_MEMEFF;
  auto kgamma = [&](CT g) -> CT {
    if (!clamp) return g;
    const CT e = CT(a.eps);
    if (g >= CT(0)) return g < e ? e : g;
    return g > -e ? -e : g;
  };
  auto xhat_of = [&](int c, CT g) -> CT {
    const CT xv = GenericIO<T, CT>::ld(xr + c);
    if (mode == BWD_LN_MEMEFF) return (xv - (bp ? GenericIO<T, CT>::ld(bp + c) : CT(0))) / kgamma(g);
    if (mode == BWD_RMS) return rs * xv;
    return rs * (xv - mu);
  };
  CT s1 = 0, s2 = 0;
  for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
    const CT g = gp ? GenericIO<T, CT>::ld(gp + c) : CT(1);
    const CT d = GenericIO<T, CT>::ld(dyr + c);
    if (mode == BWD_LN_MEMEFF) {
      const CT yb = GenericIO<T, CT>::ld(xr + c) - (bp ? GenericIO<T, CT>::ld(bp + c) : CT(0));
      s2 += d * yb;
    } else {
      s2 += d * g * xhat_of(c, g);
    }
    if (mode != BWD_RMS) s1 += d * g;
  }
  s1 = block_sum_generic<CT>(s1, lds);
  s2 = block_sum_generic<CT>(s2, lds);
  const CT inv = CT(1) / CT(a.cols);
  const CT c1 = s1 * inv, c2 = s2 * inv;
  T* dxr = static_cast<T*>(a.dx) + row * int64_t(a.cols);
  T* drr = a.dres ? static_cast<T*>(a.dres) + row * int64_t(a.cols) : nullptr;
  const T* dir = a.dx_in ? static_cast<const T*>(a.dx_in) + row * int64_t(a.cols) : nullptr;
  for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
    const CT g = gp ? GenericIO<T, CT>::ld(gp + c) : CT(1);
    const CT d = GenericIO<T, CT>::ld(dyr + c);
    CT o = rs * (d * kgamma(g) - c1 - xhat_of(c, g) * c2);
    if (dir) o += GenericIO<T, CT>::ld(dir + c);
    GenericIO<T, CT>::st(dxr + c, o);
    if (drr) GenericIO<T, CT>::st(drr + c, o);
  }
}

// dgamma[c] = sum_r dy*xhat, dbeta[c] = sum_r dy : 64 columns per block, the
// 4 waves take interleaved rows, fold through LDS.
template <typename T, typename CT>
__global__ __launch_bounds__(256)
void norm_bwd_generic_cols_kernel(NormBwdArgs a, int mode, T* dgamma, T* dbeta) {
  __shared__ CT lds[2][4][kWave];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int c = blockIdx.x * kWave + lane;
  const T* gp = static_cast<const T*>(a.gamma);
  const T* bp = static_cast<const T*>(a.beta);
  CT sg = 0, sb = 0;
  if (c < a.cols) {
    const CT g = gp ? GenericIO<T, CT>::ld(gp + c) : CT(1);
    CT kg = g;
    {
      const CT e = CT(a.eps);
      if (g >= CT(0)) kg = g < e ? e : g; else kg = g > -e ? -e : g;
    }
    const CT b = (bp && mode == BWD_LN_MEMEFF) ? GenericIO<T, CT>::ld(bp + c) : CT(0);
    for (int64_t r = w; r < a.rows; r += 4) {
      const CT d = GenericIO<T, CT>::ld(static_cast<const T*>(a.dy) + r * a.cols + c);
      const CT xv = GenericIO<T, CT>::ld(static_cast<const T*>(a.x) + r * a.cols + c);
      CT xhat;
      if (mode == BWD_LN_MEMEFF) {
        xhat = (xv - b) / kg;
      } else {
        const CT sv = a.stats_f32 ? CT(static_cast<const float*>(a.stat)[r])
                                  : GenericIO<T, CT>::ld(static_cast<const T*>(a.stat) + r);
        const CT rs = a.stat_kind == HK_STAT_VAR ? CT(1) / sqrt(sv + CT(a.eps)) : sv;
        CT mu = 0;
        if (mode == BWD_LN)
          mu = a.stats_f32 ? CT(static_cast<const float*>(a.mean)[r])
                           : GenericIO<T, CT>::ld(static_cast<const T*>(a.mean) + r);
        xhat = rs * (xv - mu);
      }
      sg += d * xhat;
      sb += d;
    }
  }
  lds[0][w][lane] = sg;
  lds[1][w][lane] = sb;
  __syncthreads();
  if (w == 0 && c < a.cols) {
    CT tg = 0, tb = 0;
    for (int i = 0; i < 4; ++i) { tg += lds[0][i][lane]; tb += lds[1][i][lane]; }
    if (dgamma) GenericIO<T, CT>::st(dgamma + c, tg);
    if (dbeta) GenericIO<T, CT>::st(dbeta + c, tb);
  }
}

struct BwdPlan {
  bool reg_path;
  int tpr, nv, rpb, grid;
  int block;
  size_t lds_bytes;
  size_t ws_bytes;
};

template <typename T>
static BwdPlan plan_norm_bwd(int64_t rows, int cols, bool aligned) {
  constexpr int VEC = VecIO<T>::N;
  BwdPlan p{};
  p.reg_path = false;
  if (!aligned || cols % VEC != 0) return p;
  const int nvec = cols / VEC;
  // column-owner kernel: the dgamma / dbeta accumulators of a thread must stay
  // in registers: 8 columns per thread by default, 16 when a thread count is forced
  const int max_nv = (tune_get(TUNE_NORM_BWD_THREADS) > 0 ? 16 : 8) / VEC;
  int tpr = tune_get(TUNE_NORM_BWD_THREADS);
  int nv;
  if (tpr > 0) {
    tpr = std::min(1024, std::max(64, (tpr + 63) / 64 * 64));
    nv = pow2_ceil((nvec + tpr - 1) / tpr);
    if (nv > max_nv) return p;
  } else {
    nv = max_nv;
    // short rows: fewer vectors per thread rather than a partly idle wavefront
    while (nv > 1 && (nvec + nv - 1) / nv < 64) nv >>= 1;
    tpr = ((nvec + nv - 1) / nv + 63) / 64 * 64;
    if (tpr > 1024) return p;
  }
  // kernels with more than one vector per thread are built for 512-thread blocks
  const int max_block = nv == 1 ? 1024 : 512;
  if (tpr > max_block) return p;
  int rpb = tune_get(TUNE_NORM_BWD_ROWS_PER_BLOCK);
  if (rpb <= 0) {
    rpb = std::max(1, max_block / tpr);
    // 512 threads already stream a whole 4096-column row per step; pairing two such groups in one
    // workgroup only adds waves to every barrier (measured 2-3 % slower than one group per workgroup)
    if (tpr >= 512) rpb = 1;
  }
  rpb = std::max(1, std::min(rpb, max_block / tpr));
  // staging buffer of the final fold must fit 64 KiB of LDS
  while (rpb > 1 && size_t(rpb) * cols * sizeof(float) > 65536) --rpb;
  int grid = tune_get(TUNE_NORM_BWD_BLOCKS);
  if (grid <= 0) grid = device_cu_count();   // one 1024-thread workgroup per CU measured fastest
  const int64_t max_useful = (rows + rpb - 1) / rpb;
  if (grid > max_useful) grid = int(max_useful);
  if (grid < 1) grid = 1;
  p.reg_path = true;
  p.tpr = tpr; p.nv = nv; p.rpb = rpb; p.grid = grid; p.block = tpr * rpb;
  p.lds_bytes = rpb > 1 ? size_t(rpb) * cols * sizeof(float) : 0;
  p.ws_bytes = size_t(2) * grid * cols * sizeof(float);
  return p;
}

template <typename T, int MODE>
static int launch_norm_bwd_nv(const NormBwdArgs& a, const BwdPlan& p, hipStream_t s) {
  dim3 grid{unsigned(p.grid)}, block{unsigned(p.block)};
  profile_before(s);
  int pf = tune_get(TUNE_NORM_BWD_PREFETCH);
  // two rows in flight where the registers allow it (RMSNorm); the LayerNorm modes carry the mean as well
  // and start spilling at depth two under the 128-register cap of 1024-thread blocks
  if (pf <= 0) pf = (MODE == BWD_RMS) ? 2 : 1;
  const bool exact = int64_t(p.nv) * p.tpr == a.nvec;
  const bool f32 = a.stats_f32 != 0;
  // statistics in the data dtype only ever come with the plain LayerNorm backward
  if (!f32 && MODE != BWD_LN) {
    set_last_error("norm_bwd: this mode keeps its statistics in float32");
    return HK_ERR_INVALID;
  }
#define HK_BWD_LAUNCH(N, P, E, F) \
  hipLaunchKernelGGL((norm_bwd_kernel<T, N, MODE, P, E, F>), grid, block, p.lds_bytes, s, a)
#define HK_BWD_EF(N, P)                                                    \
  do {                                                                     \
    if constexpr (MODE == BWD_LN) {                                        \
      if (exact && f32) HK_BWD_LAUNCH(N, P, true, true);                   \
      else if (exact) HK_BWD_LAUNCH(N, P, true, false);                    \
      else if (f32) HK_BWD_LAUNCH(N, P, false, true);                      \
      else HK_BWD_LAUNCH(N, P, false, false);                              \
    } else {                                                               \
      if (exact) HK_BWD_LAUNCH(N, P, true, true);                          \
      else HK_BWD_LAUNCH(N, P, false, true);                               \
    }                                                                      \
  } while (0)
#define HK_BWD_PF(N)                                   \
  do {                                                 \
    if (pf == 1) HK_BWD_EF(N, 1);                      \
    else if (pf == 2) HK_BWD_EF(N, 2);                 \
    else HK_BWD_EF(N, 3);                              \
  } while (0)
  switch (p.nv) {
    case 1: HK_BWD_PF(1); break;
    case 2: HK_BWD_PF(2); break;
    case 4:
      if constexpr (VecIO<T>::N == 4) { HK_BWD_PF(4); break; }
      [[fallthrough]];
    default:
      set_last_error("norm_bwd: no kernel for %d vectors per thread", p.nv);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_BWD_EF
#undef HK_BWD_PF
#undef HK_BWD_LAUNCH
  profile_after(s);
  return launch_check("norm_bwd_kernel");
}

template <typename T>
static int norm_bwd_typed(NormBwdArgs a, int mode, void* dgamma, void* dbeta, void* ws,
                          size_t ws_bytes, hipStream_t s) {
  const bool aligned = aligned16(a.dy) && aligned16(a.x) && aligned16(a.dx) && aligned16(a.gamma) &&
                       aligned16(a.beta) && aligned16(a.dx_in) && aligned16(a.dres);
  BwdPlan p = plan_norm_bwd<T>(a.rows, a.cols, aligned);
  if (!p.reg_path) {
    hipLaunchKernelGGL((norm_bwd_generic_dx_kernel<T, float>), dim3(unsigned(a.rows)), dim3(256), 0, s, a, mode);
    int rc = launch_check("norm_bwd_generic_dx_kernel");
    if (rc != HK_OK) return rc;
    if (dgamma || dbeta) {
      hipLaunchKernelGGL((norm_bwd_generic_cols_kernel<T, float>), dim3(unsigned((a.cols + 63) / 64)),
                         dim3(256), 0, s, a, mode, static_cast<T*>(dgamma), static_cast<T*>(dbeta));
      rc = launch_check("norm_bwd_generic_cols_kernel");
    }
    return rc;
  }
  const bool want_cols = dgamma != nullptr || dbeta != nullptr;
  if (want_cols) {
    HK_REQUIRE(ws != nullptr && ws_bytes >= p.ws_bytes, HK_ERR_WORKSPACE,
               "norm_bwd: workspace of %zu bytes needed, %zu given", p.ws_bytes, ws_bytes);
    HK_REQUIRE(aligned16(ws), HK_ERR_INVALID, "norm_bwd: workspace must be 16-byte aligned");
    a.part_dgamma = dgamma ? static_cast<float*>(ws) : nullptr;
    a.part_dbeta = dbeta ? static_cast<float*>(ws) + size_t(p.grid) * a.cols : nullptr;
  } else {
    a.part_dgamma = nullptr;
    a.part_dbeta = nullptr;
  }
  a.tpr = p.tpr;
  a.nvec = a.cols / VecIO<T>::N;
  int rc;
  switch (mode) {
    case BWD_LN: rc = launch_norm_bwd_nv<T, BWD_LN>(a, p, s); break;
    case BWD_RMS: rc = launch_norm_bwd_nv<T, BWD_RMS>(a, p, s); break;
    default: rc = launch_norm_bwd_nv<T, BWD_LN_MEMEFF>(a, p, s); break;
  }
  if (rc != HK_OK || !want_cols) return rc;
  hipLaunchKernelGGL((norm_bwd_finalize_kernel<T>), dim3(unsigned((a.cols + 127) / 128), 2), dim3(512), 0, s,
                     a.part_dgamma, a.part_dbeta, static_cast<T*>(dgamma), static_cast<T*>(dbeta),
                     p.grid, a.cols);
  return launch_check("norm_bwd_finalize_kernel");
}

static int norm_bwd_dispatch(int dtype, NormBwdArgs& a, int mode, void* dgamma, void* dbeta,
                             void* ws, size_t ws_bytes, hipStream_t s, const char* who) {
  HK_REQUIRE(a.rows >= 0 && a.cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  if (a.rows == 0 || a.cols == 0) return HK_OK;
  HK_REQUIRE(a.rows <= 0x7fffffffLL && a.cols <= 0x3fffffff, HK_ERR_INVALID,
             "%s: shape [%lld, %d] too large", who, (long long)a.rows, a.cols);
  HK_REQUIRE(a.dy && a.x && a.dx && a.stat, HK_ERR_INVALID, "%s: null input/output", who);
  HK_REQUIRE(mode != BWD_LN || a.mean, HK_ERR_INVALID, "%s: mean is required", who);
  a.inv_cols = 1.0f / float(a.cols);
  a.stream_store = tune_get(TUNE_STREAM_STORES) == 2 ? 0 : 1;
  switch (dtype) {
    case HK_FLOAT32: return norm_bwd_typed<float>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_BFLOAT16: return norm_bwd_typed<bf16>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_FLOAT16: return norm_bwd_typed<fp16>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_FLOAT64: {
      hipLaunchKernelGGL((norm_bwd_generic_dx_kernel<double, double>), dim3(unsigned(a.rows)), dim3(256), 0, s, a, mode);
      int rc = launch_check("norm_bwd_generic_dx_kernel<double>");
      if (rc != HK_OK) return rc;
      if (dgamma || dbeta) {
        hipLaunchKernelGGL((norm_bwd_generic_cols_kernel<double, double>), dim3(unsigned((a.cols + 63) / 64)),
                           dim3(256), 0, s, a, mode, static_cast<double*>(dgamma), static_cast<double*>(dbeta));
        rc = launch_check("norm_bwd_generic_cols_kernel<double>");
      }
      return rc;
    }
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

// ---------------------------------------------------------------------------
// Scratch memory owned by the library, for the entry point that must not
// allocate.  The array lives in the code object's global segment, so every
// device the library is loaded on holds its own copy at its own address; host
// code only ever uses the address looked up below, never the array's name.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** out) {
  int dev = -1;
  HK_CHECK_HIP(hipGetDevice(&dev));
  HK_REQUIRE(dev >= 0 && dev < kMaxDevices, HK_ERR_UNSUPPORTED,
             "static scratch: device index %d is beyond the %d devices this table holds", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    HK_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    HK_REQUIRE(p != nullptr, HK_ERR_HIP, "static scratch: symbol address is null on device %d", dev);
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return HK_OK;
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_layer_norm_fwd(int dtype, const void* x, const void* gamma, const void* beta, void* y,
                      void* mean, void* stat, int stats_dtype, int stat_kind, int64_t rows,
                      int64_t cols, float eps, hkStream_t stream) {
  HK_REQUIRE(stats_dtype == HK_FLOAT32 || stats_dtype == dtype, HK_ERR_INVALID,
             "hk_layer_norm_fwd: stats dtype %d must be fp32 or the data dtype %d", stats_dtype, dtype);
  HK_REQUIRE(stat_kind == HK_STAT_VAR || stat_kind == HK_STAT_RSTD, HK_ERR_INVALID,
             "hk_layer_norm_fwd: bad stat_kind %d", stat_kind);
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_layer_norm_fwd: cols too large");
  NormFwdArgs a{};
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y; a.mean = mean; a.stat = stat;
  a.rows = rows; a.cols = int(cols); a.eps = eps; a.is_rms = 0; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  if (dtype == HK_FLOAT64) {
    HK_REQUIRE(stats_dtype == HK_FLOAT64, HK_ERR_UNSUPPORTED,
               "hk_layer_norm_fwd: fp64 data needs fp64 statistics");
  }
  return norm_fwd_dispatch(dtype, a, as_hip(stream), "hk_layer_norm_fwd");
}

int hk_norm_bwd_workspace_bytes(int dtype, int64_t rows, int64_t cols, size_t* bytes) {
  HK_REQUIRE(bytes, HK_ERR_INVALID, "hk_norm_bwd_workspace_bytes: null output");
  HK_REQUIRE(rows >= 0 && cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID,
             "hk_norm_bwd_workspace_bytes: bad shape");
  *bytes = 0;
  if (rows == 0 || cols == 0) return HK_OK;
  BwdPlan p{};
  switch (dtype) {
    case HK_FLOAT32: p = plan_norm_bwd<float>(rows, int(cols), true); break;
    case HK_BFLOAT16: p = plan_norm_bwd<bf16>(rows, int(cols), true); break;
    case HK_FLOAT16: p = plan_norm_bwd<fp16>(rows, int(cols), true); break;
    case HK_FLOAT64: return HK_OK;
    default:
      set_last_error("hk_norm_bwd_workspace_bytes: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
  *bytes = p.reg_path ? p.ws_bytes : 0;
  return HK_OK;
}

int hk_layer_norm_bwd(int dtype, const void* dy, const void* x_or_y, const void* gamma,
                      const void* beta, const void* mean, const void* stat, int stats_dtype,
                      int stat_kind, void* dx, void* dgamma, void* dbeta, int64_t rows,
                      int64_t cols, float eps, int memory_efficient, int clamp_gamma,
                      void* workspace, size_t workspace_bytes, hkStream_t stream) {
  HK_REQUIRE(stats_dtype == HK_FLOAT32 || stats_dtype == dtype, HK_ERR_INVALID,
             "hk_layer_norm_bwd: stats dtype %d must be fp32 or the data dtype %d", stats_dtype, dtype);
  HK_REQUIRE(stat_kind == HK_STAT_VAR || stat_kind == HK_STAT_RSTD, HK_ERR_INVALID,
             "hk_layer_norm_bwd: bad stat_kind %d", stat_kind);
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_layer_norm_bwd: cols too large");
  if (dtype == HK_FLOAT64) {
    HK_REQUIRE(stats_dtype == HK_FLOAT64, HK_ERR_UNSUPPORTED,
               "hk_layer_norm_bwd: fp64 data needs fp64 statistics");
  }
  NormBwdArgs a{};
  a.dy = dy; a.x = x_or_y; a.gamma = gamma; a.beta = beta; a.mean = mean; a.stat = stat;
  a.dx = dx; a.rows = rows; a.cols = int(cols); a.eps = eps; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  a.clamp_gamma = clamp_gamma;
  return norm_bwd_dispatch(dtype, a, memory_efficient ? BWD_LN_MEMEFF : BWD_LN, dgamma, dbeta,
                           workspace, workspace_bytes, as_hip(stream), "hk_layer_norm_bwd");
}

int hk_dropout_add_ln_fwd(int itype, int rtype, int wtype, const void* x0, const void* residual,
                          const void* gamma, const void* beta, void* z, void* x_out, void* mu,
                          void* rsigma, int64_t rows, int64_t cols, float eps, int is_rms_norm,
                          hkStream_t stream) {
  HK_REQUIRE(itype == rtype && itype == wtype, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_fwd: mixed dtypes (input %d, residual %d, weight %d) are not implemented",
             itype, rtype, wtype);
  HK_REQUIRE(itype == HK_FLOAT32 || itype == HK_BFLOAT16 || itype == HK_FLOAT16, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_fwd: not implemented for dtype %d", itype);
  HK_REQUIRE(gamma != nullptr, HK_ERR_INVALID, "hk_dropout_add_ln_fwd: gamma is required");
  HK_REQUIRE(eps >= 0.f, HK_ERR_INVALID, "hk_dropout_add_ln_fwd: epsilon must be >= 0");
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_dropout_add_ln_fwd: cols too large");
  NormFwdArgs a{};
  a.x = x0; a.residual = residual; a.gamma = gamma; a.beta = beta; a.y = z; a.x_out = x_out;
  a.mean = mu; a.stat = rsigma; a.rows = rows; a.cols = int(cols); a.eps = eps;
  a.is_rms = is_rms_norm ? 1 : 0; a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1;
  return norm_fwd_dispatch(itype, a, as_hip(stream), "hk_dropout_add_ln_fwd");
}

int hk_dropout_add_ln_bwd(int itype, int rtype, int wtype, const void* dz, const void* dx_in,
                          const void* x, const void* mu, const void* rsigma, const void* gamma,
                          void* dx0, void* dresidual, void* dgamma, void* dbeta, int64_t rows,
                          int64_t cols, int is_rms_norm, void* workspace, size_t workspace_bytes,
                          hkStream_t stream) {
  HK_REQUIRE(itype == rtype && itype == wtype, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_bwd: mixed dtypes (input %d, residual %d, weight %d) are not implemented",
             itype, rtype, wtype);
  HK_REQUIRE(itype == HK_FLOAT32 || itype == HK_BFLOAT16 || itype == HK_FLOAT16, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_bwd: not implemented for dtype %d", itype);
  HK_REQUIRE(gamma != nullptr, HK_ERR_INVALID, "hk_dropout_add_ln_bwd: gamma is required");
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_dropout_add_ln_bwd: cols too large");
  NormBwdArgs a{};
  a.dy = dz; a.x = x; a.gamma = gamma; a.mean = mu; a.stat = rsigma; a.dx_in = dx_in;
  a.dx = dx0; a.dres = dresidual; a.rows = rows; a.cols = int(cols); a.eps = 0.f;
  a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1; a.clamp_gamma = 0;
  return norm_bwd_dispatch(itype, a, is_rms_norm ? BWD_RMS : BWD_LN, dgamma, dbeta, workspace,
                           workspace_bytes, as_hip(stream), "hk_dropout_add_ln_bwd");
}

int hk_dropout_add_ln_bwd_static(int itype, int rtype, int wtype, const void* dz, const void* dx_in,
                                 const void* x, const void* mu, const void* rsigma, const void* gamma,
                                 void* dx0, void* dresidual, void* dgamma, void* dbeta, int64_t rows,
                                 int64_t cols, int is_rms_norm, hkStream_t stream) {
  size_t need = 0;
  int rc = hk_norm_bwd_workspace_bytes(itype, rows, cols, &need);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(need <= kStaticScratchBytes, HK_ERR_WORKSPACE,
             "hk_dropout_add_ln_bwd_static: a [%lld, %lld] backward needs %zu bytes of column-sum partials, "
             "the library's static scratch holds %zu; use hk_dropout_add_ln_bwd with a caller workspace",
             (long long)rows, (long long)cols, need, kStaticScratchBytes);
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != HK_OK) return rc;
  // every partial row the fold kernel reads is written by this call's main kernel first: nothing in the
  // scratch has to start at zero
  return hk_dropout_add_ln_bwd(itype, rtype, wtype, dz, dx_in, x, mu, rsigma, gamma, dx0, dresidual, dgamma,
                               dbeta, rows, cols, is_rms_norm, ws, kStaticScratchBytes, stream);
}

} // extern "C"
