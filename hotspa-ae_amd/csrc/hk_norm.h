// Shared declarations of the LayerNorm / RMSNorm kernels: argument blocks, launch plans and the per-dtype entry
// points that the dispatch in hk_norm.hip calls.  The kernels themselves live in hk_norm_fwd_impl.h and
// hk_norm_bwd_impl.h and are instantiated once per storage type in hk_norm_{fwd,bwd}_{f32,bf16,f16}.hip, so
// that the types compile in parallel.
#pragma once

#include "hk_common.h"

#include <algorithm>
#include <type_traits>

namespace hk {

// Rows are `cols` elements long and lie `*_pitch` elements apart (pitch == cols for a dense array; a wider
// pitch is a column slice of a wider buffer).  Pitches are in elements of the array's type.
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
  int64_t x_pitch, res_pitch, y_pitch, xout_pitch;
  // rows on several levels (see LevelSteps), in walk order: n0 * n1 * n2 = rows; one level is n0 = rows
  int64_t n0, n1, n2;
  RowNumbering rn;
  LevelSteps x_lv, res_lv, y_lv, xout_lv;
  int cols;
  int nvec;
  float eps;
  float inv_cols;
  int is_rms;
  int stat_kind;
  int stats_f32;
};

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
  int64_t dy_pitch, x_pitch, dx_pitch, dxin_pitch, dres_pitch;
  // rows on several levels (see LevelSteps), in walk order; the walking kernel splits its walk index itself
  int64_t n0, n1, n2;
  RowNumbering rn;
  uint32_t ws0, ws1, ws2;   // the walking kernel's row stride (its grid size) split over the walk levels
  LevelSteps dy_lv, x_lv, dx_lv, dxin_lv, dres_lv;
  int cols;
  int nvec;
  int tpr;              // threads per row (multiple of 64)
  float eps;
  float inv_cols;
  int stat_kind;
  int stats_f32;
  int clamp_gamma;
};

struct BwdPlan {
  bool reg_path;
  int tpr, nv, rpb, grid;
  int block;
  size_t lds_bytes;
  size_t ws_bytes;
};

static inline int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <typename T>
__device__ __forceinline__ void store_stat(void* base, int64_t row, float v, int stats_f32) {
  if (base == nullptr) return;
  if (stats_f32) static_cast<float*>(base)[row] = v;
  else Cvt<T>::store(static_cast<T*>(base) + row, v);
}

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

// Per-type entry points (T = float, bf16, fp16), defined by the explicit instantiations.
template <typename T> int norm_fwd_typed(NormFwdArgs a, hipStream_t s);
template <typename T> BwdPlan plan_norm_bwd(int64_t rows, int cols, bool aligned);
template <typename T> int norm_bwd_typed(NormBwdArgs a, int mode, void* dgamma, void* dbeta, void* ws,
                                          size_t ws_bytes, hipStream_t s);
// double precision: one workgroup per row, arithmetic in double (with the fp32 instantiations)
int norm_fwd_f64(const NormFwdArgs& a, hipStream_t s);
int norm_bwd_f64(const NormBwdArgs& a, int mode, void* dgamma, void* dbeta, hipStream_t s);

} // namespace hk
