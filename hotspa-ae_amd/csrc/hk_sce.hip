// Fused softmax cross-entropy forward / backward for gfx950 (sparse int64
// labels with an ignored index, and dense labels).
//
// A logits row is read from HBM once and kept in registers; each thread folds
// its elements into a (max, sum-of-exp) pair, pairs are merged online across
// lanes (DPP) and waves (LDS).  Forward writes one loss per row; backward
// rescales the stored exponentials into (softmax - onehot) * grad_loss and
// writes the row once.  Rows whose label equals the ignored index are not read
// at all: loss 0 / a zero gradient row is written.
#include "hk_common.h"

#include <algorithm>

namespace hk {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegInf = -__builtin_huge_valf();

struct SceArgs {
  const void* logits;
  const int64_t* labels;   // sparse
  const void* dlabels;     // dense labels (same shape as logits)
  const void* grad_loss;   // backward
  void* out;               // forward: loss [rows]; backward: dlogits
  int64_t rows;
  // elements between the starts of consecutive rows of logits / dense labels / dlogits (0 = dense: cols)
  int64_t x_pitch, lab_pitch, out_pitch;
  // rows on several levels (see LevelSteps); one level: n0 = rows.  labels, losses, per-row gradients and
  // statistics are dense [rows] arrays and take the row's number
  int64_t n0, n1, n2;
  RowNumbering rn;
  LevelSteps x_lv, lab_lv, out_lv;
  int cols;
  int nvec;
  int64_t ignored_index;
  // sparse forward on a column shard [vocab_start, vocab_start + cols) of a wider row: instead of a loss,
  // stats[0..rows) = the shard's row maximum, stats[rows..2 rows) = sum of exp(x - that maximum),
  // stats[2 rows..3 rows) = the logit at the label when the label falls into the shard, else 0
  float* stats;
  int64_t vocab_start;
  // backward of a reduced loss: grad_loss holds ONE value (the gradient of the mean / sum) and every row uses
  // round_T(that value * grad_scale), which is what broadcasting it times 1/rows into a [rows] array of the
  // storage type first would have handed to this kernel
  int grad_scalar;
  double grad_scale;
};

template <typename T, typename CT>
__device__ __forceinline__ CT sce_row_grad(const SceArgs& a, int64_t row) {
  const T* gp = static_cast<const T*>(a.grad_loss);
  if (!a.grad_scalar) return CT(Cvt<T>::load(gp + row));
  T rounded;
  Cvt<T>::store(&rounded, CT(Cvt<T>::load(gp)) * CT(a.grad_scale));
  return CT(Cvt<T>::load(&rounded));
}

// i0: the row's place within the innermost level (blockIdx.y / z are the outer levels); row: its number
template <bool WAVE_ROW>
__device__ __forceinline__ void row_coords(const SceArgs& a, int& tpr, int& t, int64_t& i0, int64_t& row, int& nwaves) {
  tpr = WAVE_ROW ? kWave : int(blockDim.x);
  t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  i0 = WAVE_ROW ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index() : int64_t(blockIdx.x);
  row = dense_row_index(i0, a.rn);
  nwaves = WAVE_ROW ? 1 : int(blockDim.x >> 6);
}

// ------------------------------- sparse forward ----------------------------
template <typename T, int NV, bool WAVE_ROW>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024)
void sce_sparse_fwd_kernel(SceArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves * 3];
  int tpr, t, nwaves;
  int64_t i0, row;
  row_coords<WAVE_ROW>(a, tpr, t, i0, row, nwaves);
  if (WAVE_ROW && i0 >= a.n0) return;

  T* loss = static_cast<T*>(a.out);
  const int64_t label = a.labels[row];
  if (label == a.ignored_index) {          // uniform over the row's threads
    if (t == 0) {
      if (a.stats) {
        a.stats[row] = kNegInf;
        a.stats[a.rows + row] = 0.f;
        a.stats[2 * a.rows + row] = 0.f;
      } else {
        Cvt<T>::store(loss + row, 0.f);
      }
    }
    return;
  }
  const T* xr = static_cast<const T*>(a.logits) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
  // slots past the row's end hold -inf: they change neither the maximum nor the sum
  float f[NV * VEC];
  {
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
#pragma unroll
    for (int i = 0; i < NV; ++i) VecIO<T>::unpack(raw[i], &f[i * VEC]);
  }
  float m = f[0];
  static_assert((NV * VEC) % 2 == 0, "pairs of elements per max3");
  m = fmaxf(m, f[1]);
#pragma unroll
  for (int e = 2; e < NV * VEC; e += 2) m = max3(m, f[e], f[e + 1]);
  // ml: this thread's maximum in the log2 domain, rounded once (see OnlineSoftmaxTuple)
  const float ml = (m == kNegInf) ? 0.f : m * kLog2e;
  // four independent chains: the exponential unit's latency is not serialised behind one accumulator
  float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int e = 0; e < NV * VEC; ++e) s4[e & 3] += __builtin_amdgcn_exp2f(fmaf(f[e], kLog2e, -ml));
  const float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
  MaxSumMaxTuple p;
  p.v[0] = (m == kNegInf) ? kNegInf : ml; p.v[1] = s; p.v[2] = m;
  p = WAVE_ROW ? wave_allreduce_tuple(p) : group_allreduce_tuple(p, red, 0, nwaves);
  if (t == 0 && a.stats) {
    const float M = p.v[2];
    // sum exp(x - M) = S * 2^(ML - M * log2e)
    a.stats[row] = M;
    a.stats[a.rows + row] = (M == kNegInf) ? 0.f : p.v[1] * __builtin_amdgcn_exp2f(-fmaf(M, kLog2e, -p.v[0]));
    const int64_t local = label - a.vocab_start;
    a.stats[2 * a.rows + row] = (local >= 0 && local < a.cols) ? Cvt<T>::load(xr + local) : 0.f;
  } else if (t == 0) {
    float r;
    if (label >= 0 && label < a.cols) {
      const float xl = Cvt<T>::load(xr + label);
      // sum exp(x - M) = S * 2^(ML - M * log2e); the fma recovers the rounding of ML exactly
      const float M = p.v[2];
      const float log2s = __builtin_amdgcn_logf(p.v[1]) - fmaf(M, kLog2e, -p.v[0]);
      // M - xl first: the difference of two logits is (nearly) exact however large their common offset is, and
      // the sum then rounds at the size of the loss, not of the logits
      r = log2s * kLn2 + (M - xl);
    } else {
      r = __builtin_nanf("");  // label outside [0, cols): no logit to gather
    }
    Cvt<T>::store(loss + row, r);
  }
}

// ------------------------------- sparse backward ---------------------------
// A 1024-thread workgroup is four wavefronts on every SIMD: two such workgroups fit a compute unit only at the
// full eight wavefronts per SIMD, i.e. at 64 registers or fewer.  The second launch bound asks the compiler for
// that; without it the kernel came out at 68 registers and ran with one workgroup per compute unit (448 us
// instead of 345 us at 16384 x 32000 bf16).  Eight fp32 vectors per thread do not fit 64 registers and keep the
// looser bound.
template <typename T, int NV>
constexpr int sce_min_waves(bool wave_row) { return wave_row ? 1 : (sizeof(T) == 4 && NV == 8 ? 4 : 8); }

template <typename T, int NV, bool WAVE_ROW>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024, (sce_min_waves<T, NV>(WAVE_ROW)))
void sce_sparse_bwd_kernel(SceArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves * 2];
  int tpr, t, nwaves;
  int64_t i0, row;
  row_coords<WAVE_ROW>(a, tpr, t, i0, row, nwaves);
  if (WAVE_ROW && i0 >= a.n0) return;

  T* dxr = static_cast<T*>(a.out) + i0 * a.out_pitch + outer_level_offset(a.out_lv);
  const int64_t label = a.labels[row];
  if (label == a.ignored_index) {
    const u32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * tpr + t;
      if (v < a.nvec) {
        st16_stream(dxr + v * VEC, z);
      }
    }
    return;
  }
  const T* xr = static_cast<const T*>(a.logits) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
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
  const float g = sce_row_grad<T, float>(a, row);
  float e[NV * VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i) VecIO<T>::unpack(raw[i], &e[i * VEC]);
  static_assert((NV * VEC) % 2 == 0, "pairs of elements per max3");
  float m = fmaxf(e[0], e[1]);
#pragma unroll
  for (int k = 2; k < NV * VEC; k += 2) m = max3(m, e[k], e[k + 1]);
  const float ml = (m == kNegInf) ? 0.f : m * kLog2e;
  // four independent chains, as in the forward kernel
  float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < NV * VEC; ++k) {
    e[k] = __builtin_amdgcn_exp2f(fmaf(e[k], kLog2e, -ml));
    s4[k & 3] += e[k];
  }
  const float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
  MaxSumTuple p;
  p.v[0] = (m == kNegInf) ? kNegInf : ml; p.v[1] = s;
  p = WAVE_ROW ? wave_allreduce_tuple(p) : group_allreduce_tuple(p, red, 0, nwaves);
  const float ML = (p.v[0] == kNegInf) ? 0.f : p.v[0];
  const float scale = __builtin_amdgcn_exp2f(ml - ML) / p.v[1] * g;
  const int lvec = int(label / VEC), lsub = int(label - int64_t(lvec) * VEC);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    if (v < a.nvec) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) e[i * VEC + j] *= scale;
      if (label >= 0 && v == lvec) {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          if (j == lsub) e[i * VEC + j] -= g;
      }
      const u32x4 o = VecIO<T>::pack(&e[i * VEC]);
      st16_stream(dxr + v * VEC, o);
    }
  }
}

// ------------------------------- dense labels ------------------------------
// loss = (M + log S) * sum(l) - sum(l * x);  dx = (softmax - l) * g
template <typename T, int NV, bool WAVE_ROW, bool BWD>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024, (sce_min_waves<T, NV>(WAVE_ROW)))
void sce_dense_kernel(SceArgs a) {
  constexpr int VEC = VecIO<T>::N;
  __shared__ float red[kMaxWaves * 3];
  __shared__ float red2[kMaxWaves * 2];
  int tpr, t, nwaves;
  int64_t i0, row;
  row_coords<WAVE_ROW>(a, tpr, t, i0, row, nwaves);
  if (WAVE_ROW && i0 >= a.n0) return;

  const T* xr = static_cast<const T*>(a.logits) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
  const T* lr = static_cast<const T*>(a.dlabels) + i0 * a.lab_pitch + outer_level_offset(a.lab_lv);
  u32x4 rx[NV], rl[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * tpr + t;
    rx[i] = u32x4{0, 0, 0, 0};
    rl[i] = u32x4{0, 0, 0, 0};
    if (v < a.nvec) { rx[i] = ld16(xr + v * VEC); rl[i] = ld16(lr + v * VEC); }
  }
  float m = kNegInf;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (i * tpr + t < a.nvec) {
      float f[VEC];
      VecIO<T>::unpack(rx[i], f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) m = fmaxf(m, f[j]);
    }
  }
  const float ml = (m == kNegInf) ? 0.f : m * kLog2e;
  float s = 0.f;
  SumTuple<2> ls;
  ls.v[0] = 0.f; ls.v[1] = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (i * tpr + t < a.nvec) {
      float f[VEC], l[VEC];
      VecIO<T>::unpack(rx[i], f);
      VecIO<T>::unpack(rl[i], l);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s += __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -ml));
        if constexpr (!BWD) { ls.v[0] += l[j]; ls.v[1] = fmaf(l[j], f[j], ls.v[1]); }
      }
    }
  }
  MaxSumMaxTuple p;
  p.v[0] = (m == kNegInf) ? kNegInf : ml; p.v[1] = s; p.v[2] = m;
  p = WAVE_ROW ? wave_allreduce_tuple(p) : group_allreduce_tuple(p, red, 0, nwaves);
  if constexpr (!BWD) {
    ls = WAVE_ROW ? wave_allreduce_tuple(ls) : group_allreduce_tuple(ls, red2, 0, nwaves);
    if (t == 0) {
      const float M = p.v[2];
      const float log2s = __builtin_amdgcn_logf(p.v[1]) - fmaf(M, kLog2e, -p.v[0]);
      const float lse = log2s * kLn2 + M;
      Cvt<T>::store(static_cast<T*>(a.out) + row, lse * ls.v[0] - ls.v[1]);
    }
  } else {
    const float g = sce_row_grad<T, float>(a, row);
    const float ML = (p.v[0] == kNegInf) ? 0.f : p.v[0];
    const float inv = 1.0f / p.v[1];
    T* dxr = static_cast<T*>(a.out) + i0 * a.out_pitch + outer_level_offset(a.out_lv);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * tpr + t;
      if (v < a.nvec) {
        float f[VEC], l[VEC];
        VecIO<T>::unpack(rx[i], f);
        VecIO<T>::unpack(rl[i], l);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          f[j] = (__builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -ML)) * inv - l[j]) * g;
        const u32x4 o = VecIO<T>::pack(f);
        st16_stream(dxr + v * VEC, o);
      }
    }
  }
}

// ------------------------------- fallback ----------------------------------
// Any cols / alignment / dtype: one workgroup per row, strided passes.
template <typename T, typename CT>
struct SceIO {
  static __device__ __forceinline__ CT ld(const T* p) { return CT(Cvt<T>::load(p)); }
  static __device__ __forceinline__ void st(T* p, CT v) { Cvt<T>::store(p, v); }
};
template <typename CT> __device__ __forceinline__ CT sce_exp(CT v);
template <> __device__ __forceinline__ float sce_exp<float>(float v) { return __builtin_amdgcn_exp2f(v * kLog2e); }
template <> __device__ __forceinline__ double sce_exp<double>(double v) { return exp(v); }
template <typename CT> __device__ __forceinline__ CT sce_log(CT v);
template <> __device__ __forceinline__ float sce_log<float>(float v) { return __builtin_amdgcn_logf(v) * kLn2; }
template <> __device__ __forceinline__ double sce_log<double>(double v) { return log(v); }

template <typename CT>
__device__ __forceinline__ CT sce_block_reduce(CT v, CT* lds, bool is_max) {
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

// MODE 0: sparse fwd, 1: sparse bwd, 2: dense fwd, 3: dense bwd
template <typename T, typename CT, int MODE>
__global__ __launch_bounds__(256)
void sce_generic_kernel(SceArgs a) {
  __shared__ CT lds[256];
  const int64_t i0 = blockIdx.x;
  const int64_t row = dense_row_index(i0, a.rn);
  const int64_t cols = a.cols;
  const T* xr = static_cast<const T*>(a.logits) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
  int64_t label = 0;
  if (MODE < 2) {
    label = a.labels[row];
    if (label == a.ignored_index) {
      if (MODE == 0) {
        if (threadIdx.x == 0) {
          if (a.stats) {
            a.stats[row] = kNegInf;
            a.stats[a.rows + row] = 0.f;
            a.stats[2 * a.rows + row] = 0.f;
          } else {
            SceIO<T, CT>::st(static_cast<T*>(a.out) + row, CT(0));
          }
        }
      } else {
        T* dxr = static_cast<T*>(a.out) + i0 * a.out_pitch + outer_level_offset(a.out_lv);
        for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) SceIO<T, CT>::st(dxr + c, CT(0));
      }
      return;
    }
  }
  CT m = -__builtin_huge_val();
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
    const CT v = SceIO<T, CT>::ld(xr + c);
    m = v > m ? v : m;
  }
  m = sce_block_reduce<CT>(m, lds, true);
  CT s = 0;
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) s += sce_exp<CT>(SceIO<T, CT>::ld(xr + c) - m);
  s = sce_block_reduce<CT>(s, lds, false);
  if (MODE == 0 && a.stats) {
    if (threadIdx.x == 0) {
      const int64_t local = label - a.vocab_start;
      a.stats[row] = float(m);
      a.stats[a.rows + row] = float(s);
      a.stats[2 * a.rows + row] = (local >= 0 && local < cols) ? float(SceIO<T, CT>::ld(xr + local)) : 0.f;
    }
  } else if (MODE == 0) {
    if (threadIdx.x == 0) {
      CT r;
      if (label >= 0 && label < cols) r = sce_log<CT>(s) + (m - SceIO<T, CT>::ld(xr + label));
      else r = CT(__builtin_nanf(""));
      SceIO<T, CT>::st(static_cast<T*>(a.out) + row, r);
    }
  } else if (MODE == 2) {
    const T* lr = static_cast<const T*>(a.dlabels) + i0 * a.lab_pitch + outer_level_offset(a.lab_lv);
    CT sl = 0, slx = 0;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      const CT l = SceIO<T, CT>::ld(lr + c);
      sl += l;
      slx += l * SceIO<T, CT>::ld(xr + c);
    }
    sl = sce_block_reduce<CT>(sl, lds, false);
    slx = sce_block_reduce<CT>(slx, lds, false);
    if (threadIdx.x == 0)
      SceIO<T, CT>::st(static_cast<T*>(a.out) + row, (sce_log<CT>(s) + m) * sl - slx);
  } else {
    const CT g = sce_row_grad<T, CT>(a, row);
    const CT inv = CT(1) / s;
    T* dxr = static_cast<T*>(a.out) + i0 * a.out_pitch + outer_level_offset(a.out_lv);
    const T* lr = MODE == 3 ? static_cast<const T*>(a.dlabels) + i0 * a.lab_pitch + outer_level_offset(a.lab_lv) : nullptr;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      CT pr = sce_exp<CT>(SceIO<T, CT>::ld(xr + c) - m) * inv;
      if (MODE == 1) pr = (c == label) ? (pr * g - g) : pr * g;
      else pr = (pr - SceIO<T, CT>::ld(lr + c)) * g;
      SceIO<T, CT>::st(dxr + c, pr);
    }
  }
}

static inline int pow2_ceil_sce(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

static bool pick_sce_shape(int nvec, int max_nv_wave, int max_nv, int* threads, int* nv) {
  const int forced = tune_get(TUNE_SCE_THREADS);
  if (forced > 0) {
    int t = std::min(1024, std::max(64, (forced + 63) / 64 * 64));
    int n = pow2_ceil_sce((nvec + t - 1) / t);
    if (n > max_nv) return false;
    *threads = t; *nv = n;
    return true;
  }
  if (nvec <= 64 * max_nv_wave) {
    *threads = 64;
    *nv = pow2_ceil_sce((nvec + 63) / 64);
    return true;
  }
  // long rows, measured at 32000 bf16 columns: the widest vector count the
  // kernel is built for wins (512 threads x 8 vectors beat 1024 x 4 forward)
  for (int n = max_nv; n >= 1; n >>= 1) {
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 1024 && (t >= 256 || n == 1)) { *threads = t; *nv = n; return true; }
  }
  for (int n = 1; n <= max_nv; n <<= 1) {
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if (t <= 1024) { *threads = t; *nv = n; return true; }
  }
  return false;
}

// MODE as in sce_generic_kernel
template <typename T, int MODE, bool WAVE_ROW>
static int launch_sce_nv(const SceArgs& a, int nv, dim3 grid, dim3 block, hipStream_t s) {
#define HK_SCE_LAUNCH(N)                                                                         \
  do {                                                                                           \
    if constexpr (MODE == 0) HK_LAUNCH((sce_sparse_fwd_kernel<T, N, WAVE_ROW>), grid, block, 0, s, a); \
    else if constexpr (MODE == 1) HK_LAUNCH((sce_sparse_bwd_kernel<T, N, WAVE_ROW>), grid, block, 0, s, a); \
    else if constexpr (MODE == 2) HK_LAUNCH((sce_dense_kernel<T, N, WAVE_ROW, false>), grid, block, 0, s, a); \
    else HK_LAUNCH((sce_dense_kernel<T, N, WAVE_ROW, true>), grid, block, 0, s, a);       \
  } while (0)
  profile_before(s);
  switch (nv) {
    case 1: HK_SCE_LAUNCH(1); break;
    case 2: HK_SCE_LAUNCH(2); break;
    case 4: HK_SCE_LAUNCH(4); break;
    case 8:
      if constexpr (MODE == 0 || VecIO<T>::N == 4) { HK_SCE_LAUNCH(8); break; }
      [[fallthrough]];
    default:
      set_last_error("softmax cross-entropy: no kernel for %d vectors per thread", nv);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_SCE_LAUNCH
  profile_after(s);
  return launch_check("sce kernel");
}

template <typename T, int MODE>
static int sce_typed(SceArgs a, hipStream_t s) {
  constexpr int VEC = VecIO<T>::N;
  auto steps_ok = [](int64_t pitch, const LevelSteps& l) { return pitch % VEC == 0 && l.p1 % VEC == 0 && l.p2 % VEC == 0; };
  const bool vec_ok = a.cols % VEC == 0 && aligned16(a.logits) && aligned16(a.dlabels) &&
                      (MODE == 0 || MODE == 2 || (aligned16(a.out) && steps_ok(a.out_pitch, a.out_lv))) &&
                      steps_ok(a.x_pitch, a.x_lv) && (MODE < 2 || steps_ok(a.lab_pitch, a.lab_lv));
  a.nvec = a.cols / VEC;
  // sparse forward only keeps the packed row; the others keep 32 floats or two rows
  const int max_nv = (MODE == 0) ? 8 : 32 / VEC;
  const int max_nv_wave = (MODE == 0) ? 8 : 32 / VEC;
  int threads = 0, nv = 0;
  if (vec_ok && pick_sce_shape(a.nvec, max_nv_wave, max_nv, &threads, &nv)) {
    if (threads == 64) {
      dim3 grid(unsigned((a.n0 + 3) / 4), unsigned(a.n1), unsigned(a.n2)), block(256);
      return launch_sce_nv<T, MODE, true>(a, nv, grid, block, s);
    }
    dim3 grid{unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)}, block{unsigned(threads)};
    return launch_sce_nv<T, MODE, false>(a, nv, grid, block, s);
  }
  HK_LAUNCH((sce_generic_kernel<T, float, MODE>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)), dim3(256), 0,
            s, a);
  return launch_check("sce_generic_kernel");
}

template <int MODE>
static int sce_dispatch(int dtype, SceArgs& a, hipStream_t s, const char* who) {
  HK_REQUIRE(a.rows >= 0 && a.cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  if (a.rows == 0) return HK_OK;
  HK_REQUIRE(a.cols > 0, HK_ERR_INVALID, "%s: rows without classes", who);
  HK_REQUIRE(a.rows <= 0x7fffffffLL, HK_ERR_INVALID, "%s: too many rows", who);
  HK_REQUIRE(a.logits && a.out, HK_ERR_INVALID, "%s: null input/output", who);
  HK_REQUIRE(MODE >= 2 || a.labels, HK_ERR_INVALID, "%s: null labels", who);
  HK_REQUIRE(MODE < 2 || a.dlabels, HK_ERR_INVALID, "%s: null labels", who);
  HK_REQUIRE((MODE & 1) == 0 || a.grad_loss, HK_ERR_INVALID, "%s: null grad_loss", who);
  if (a.x_pitch == 0) a.x_pitch = a.cols;
  if (a.lab_pitch == 0) a.lab_pitch = a.cols;
  if (a.out_pitch == 0) a.out_pitch = a.cols;
  if (a.n0 == 0) { a.n0 = a.rows; a.n1 = a.n2 = 1; a.rn = RowNumbering{1, 0, 0}; }   // one level
  HK_REQUIRE(a.n0 == 1 || (a.x_pitch >= a.cols && a.lab_pitch >= a.cols && a.out_pitch >= a.cols), HK_ERR_INVALID,
             "%s: a row pitch is smaller than the %d columns of a row", who, a.cols);
  switch (dtype) {
    case HK_FLOAT32: return sce_typed<float, MODE>(a, s);
    case HK_BFLOAT16: return sce_typed<bf16, MODE>(a, s);
    case HK_FLOAT16: return sce_typed<fp16, MODE>(a, s);
    case HK_FLOAT64:
      HK_LAUNCH((sce_generic_kernel<double, double, MODE>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)),
                dim3(256), 0, s, a);
      return launch_check("sce_generic_kernel<double>");
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_sce_sparse_fwd(int dtype, const void* logits, const int64_t* labels, void* loss, int64_t rows,
                      int64_t cols, int64_t ignored_index, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_sparse_fwd: cols too large");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.out = loss; a.rows = rows; a.cols = int(cols);
  a.ignored_index = ignored_index;
  return sce_dispatch<0>(dtype, a, as_hip(stream), "hk_sce_sparse_fwd");
}

// logits_steps / out_steps (out_steps may be null): the operands' steps in the rows' own order
static int sce_levels(SceArgs& a, const int64_t level_rows[3], const int64_t* logits_steps, const int64_t* out_steps,
                      const char* who) {
  HK_REQUIRE(level_rows, HK_ERR_INVALID, "%s: null level_rows", who);
  const int64_t n0 = level_rows[0], n1 = level_rows[1], n2 = level_rows[2];
  HK_REQUIRE(n0 >= 0 && n1 >= 0 && n2 >= 0, HK_ERR_INVALID, "%s: negative level count", who);
  a.rows = 0;
  if (n0 == 0 || n1 == 0 || n2 == 0) return HK_OK;
  HK_REQUIRE(n0 <= 0x7fffffffLL && n0 * n1 <= 0x7fffffffLL && n0 * n1 * n2 <= 0x7fffffffLL, HK_ERR_INVALID,
             "%s: too many rows", who);
  a.rows = n0 * n1 * n2;
  int64_t key[3] = {0, 0, 0};
  for (int k = 0; k < 3; ++k) key[k] = logits_steps[k] + (out_steps ? out_steps[k] : 0);
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  HK_REQUIRE(walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)n0, (long long)n1, (long long)n2);
  a.n0 = w.n[0]; a.n1 = w.n[1]; a.n2 = w.n[2]; a.rn = w.rn;
  walk_steps(w, logits_steps, &a.x_pitch, &a.x_lv);
  if (out_steps) walk_steps(w, out_steps, &a.out_pitch, &a.out_lv);
  return HK_OK;
}

int hk_sce_sparse_fwd_strided_rows(int dtype, const void* logits, const int64_t logits_steps[3],
                                   const int64_t* labels, void* loss, const int64_t level_rows[3], int64_t cols,
                                   int64_t ignored_index, hkStream_t stream) {
  const char* who = "hk_sce_sparse_fwd_strided_rows";
  HK_REQUIRE(logits_steps, HK_ERR_INVALID, "%s: null steps", who);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  SceArgs a{};
  int rc = sce_levels(a, level_rows, logits_steps, nullptr, who);
  if (rc != HK_OK) return rc;
  a.logits = logits; a.labels = labels; a.out = loss; a.cols = int(cols);
  a.ignored_index = ignored_index;
  return sce_dispatch<0>(dtype, a, as_hip(stream), who);
}

int hk_sce_sparse_bwd_strided_rows(int dtype, const void* logits, const int64_t logits_steps[3],
                                   const int64_t* labels, const void* grad_loss, void* dlogits,
                                   const int64_t dlogits_steps[3], const int64_t level_rows[3], int64_t cols,
                                   int64_t ignored_index, hkStream_t stream) {
  const char* who = "hk_sce_sparse_bwd_strided_rows";
  HK_REQUIRE(logits_steps && dlogits_steps, HK_ERR_INVALID, "%s: null steps", who);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  SceArgs a{};
  int rc = sce_levels(a, level_rows, logits_steps, dlogits_steps, who);
  if (rc != HK_OK) return rc;
  a.logits = logits; a.labels = labels; a.grad_loss = grad_loss; a.out = dlogits; a.cols = int(cols);
  a.ignored_index = ignored_index;
  return sce_dispatch<1>(dtype, a, as_hip(stream), who);
}

int hk_sce_sparse_fwd_pitched(int dtype, const void* logits, int64_t logits_pitch, const int64_t* labels,
                              void* loss, int64_t rows, int64_t cols, int64_t ignored_index, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_sparse_fwd_pitched: cols too large");
  HK_REQUIRE(logits_pitch > 0, HK_ERR_INVALID, "hk_sce_sparse_fwd_pitched: a row pitch must be positive");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.out = loss; a.rows = rows; a.cols = int(cols);
  a.x_pitch = logits_pitch; a.ignored_index = ignored_index;
  return sce_dispatch<0>(dtype, a, as_hip(stream), "hk_sce_sparse_fwd_pitched");
}

int hk_sce_sparse_bwd_pitched(int dtype, const void* logits, int64_t logits_pitch, const int64_t* labels,
                              const void* grad_loss, void* dlogits, int64_t dlogits_pitch, int64_t rows,
                              int64_t cols, int64_t ignored_index, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_sparse_bwd_pitched: cols too large");
  HK_REQUIRE(logits_pitch > 0 && dlogits_pitch > 0, HK_ERR_INVALID,
             "hk_sce_sparse_bwd_pitched: a row pitch must be positive");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.grad_loss = grad_loss; a.out = dlogits; a.rows = rows;
  a.cols = int(cols); a.x_pitch = logits_pitch; a.out_pitch = dlogits_pitch; a.ignored_index = ignored_index;
  return sce_dispatch<1>(dtype, a, as_hip(stream), "hk_sce_sparse_bwd_pitched");
}

int hk_vocab_parallel_ce_stats(int dtype, const void* logits, const int64_t* labels, float* stats, int64_t rows,
                               int64_t cols, int64_t vocab_start, int64_t ignored_index, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_vocab_parallel_ce_stats: cols too large");
  HK_REQUIRE(rows == 0 || stats != nullptr, HK_ERR_INVALID, "hk_vocab_parallel_ce_stats: null output");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.out = stats; a.rows = rows; a.cols = int(cols);
  a.ignored_index = ignored_index; a.stats = stats; a.vocab_start = vocab_start;
  return sce_dispatch<0>(dtype, a, as_hip(stream), "hk_vocab_parallel_ce_stats");
}

int hk_sce_sparse_bwd(int dtype, const void* logits, const int64_t* labels, const void* grad_loss,
                      void* dlogits, int64_t rows, int64_t cols, int64_t ignored_index,
                      hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_sparse_bwd: cols too large");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.grad_loss = grad_loss; a.out = dlogits; a.rows = rows;
  a.cols = int(cols); a.ignored_index = ignored_index;
  return sce_dispatch<1>(dtype, a, as_hip(stream), "hk_sce_sparse_bwd");
}

int hk_sce_sparse_bwd_reduced(int dtype, const void* logits, const int64_t* labels, const void* grad_output,
                              double scale, void* dlogits, int64_t rows, int64_t cols, int64_t ignored_index,
                              hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_sparse_bwd_reduced: cols too large");
  SceArgs a{};
  a.logits = logits; a.labels = labels; a.grad_loss = grad_output; a.out = dlogits; a.rows = rows;
  a.cols = int(cols); a.ignored_index = ignored_index;
  a.grad_scalar = 1;
  a.grad_scale = round_to_dtype(dtype, scale);
  return sce_dispatch<1>(dtype, a, as_hip(stream), "hk_sce_sparse_bwd_reduced");
}

int hk_sce_dense_bwd_reduced(int dtype, const void* logits, const void* labels, const void* grad_output,
                             double scale, void* dlogits, int64_t rows, int64_t cols, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_dense_bwd_reduced: cols too large");
  SceArgs a{};
  a.logits = logits; a.dlabels = labels; a.grad_loss = grad_output; a.out = dlogits; a.rows = rows;
  a.cols = int(cols);
  a.grad_scalar = 1;
  a.grad_scale = round_to_dtype(dtype, scale);
  return sce_dispatch<3>(dtype, a, as_hip(stream), "hk_sce_dense_bwd_reduced");
}

int hk_sce_dense_fwd(int dtype, const void* logits, const void* labels, void* loss, int64_t rows,
                     int64_t cols, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_dense_fwd: cols too large");
  SceArgs a{};
  a.logits = logits; a.dlabels = labels; a.out = loss; a.rows = rows; a.cols = int(cols);
  return sce_dispatch<2>(dtype, a, as_hip(stream), "hk_sce_dense_fwd");
}

int hk_sce_dense_bwd(int dtype, const void* logits, const void* labels, const void* grad_loss,
                     void* dlogits, int64_t rows, int64_t cols, hkStream_t stream) {
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_sce_dense_bwd: cols too large");
  SceArgs a{};
  a.logits = logits; a.dlabels = labels; a.grad_loss = grad_loss; a.out = dlogits; a.rows = rows;
  a.cols = int(cols);
  return sce_dispatch<3>(dtype, a, as_hip(stream), "hk_sce_dense_bwd");
}

} // extern "C"
