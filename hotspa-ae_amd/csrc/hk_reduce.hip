// Reduce sum / mean / max / min / product over arbitrary axes for gfx950.
//
// The host merges neighbouring dimensions of the same kind (reduced / kept)
// that are contiguous in memory, then picks one of three kernels:
//   inner   [rows, C] -> [rows]   : the reduced extent is the unit-stride one;
//           a wavefront or workgroup streams a row with 128-bit loads, DPP +
//           LDS fold.  Long rows are split over several workgroups.
//   outer   [B, R, C] -> [B, C]   : the kept extent is the unit-stride one;
//           every lane owns one 128-bit column vector, the waves of a
//           workgroup take runs of consecutive rows, rows are split over many
//           workgroups, fp32 partials are folded by a second small launch
//           (folding inside the first launch, by the workgroup that arrives
//           last at a per-tile counter, was built and measured slower: 86 us
//           per call with device-scope fences, 44.5 us with device-scope
//           accesses instead of fences, against 43.1 us for two launches).
//   generic any strided layout    : one thread per output element.
// bf16 / fp16 accumulate in fp32; mean multiplies the final sum by
// float(1 / reduce_num).  Every kernel takes the reduction (identity + combine)
// as a type, so all five share the same planning and memory access.
#include "hk_common.h"

#include <algorithm>
#include <limits>
#include <type_traits>
#include <vector>

namespace hk {

// ---------------------------------------------------------------------------
// element access for the scalar paths
// ---------------------------------------------------------------------------
template <typename T> struct AccOf { using type = T; };
template <> struct AccOf<bf16> { using type = float; };
template <> struct AccOf<fp16> { using type = float; };
template <> struct AccOf<bool> { using type = int64_t; };

template <typename T, typename ACC>
__device__ __forceinline__ ACC ld_acc(const T* p) {
  if constexpr (std::is_same<T, bf16>::value || std::is_same<T, fp16>::value) return ACC(Cvt<T>::load(p));
  else return ACC(*p);
}
template <typename T, typename ACC>
__device__ __forceinline__ void st_acc(T* p, ACC v) {
  if constexpr (std::is_same<T, bf16>::value || std::is_same<T, fp16>::value) Cvt<T>::store(p, float(v));
  else *p = T(v);
}
// sum -> output value (mean applies the fp32 factor, ReduceMean.cu:9-22)
template <typename ACC>
__device__ __forceinline__ ACC project(ACC v, float factor, int is_mean) {
  if (!is_mean) return v;
  if constexpr (std::is_floating_point<ACC>::value) return v * ACC(factor);
  else return ACC(float(v) * factor);
}

// The reductions: identity element and combine.  Max / min return a NaN as soon as one operand is a NaN,
// as (isnan(a) || a > b) ? a : b does in the reference (ReduceMax.cu:10-14, ReduceMin.cu:10-14); their
// identities are -inf / +inf (the integer type's extremes for integers); the product starts from 1
// (ReduceProd.cu:8-24).
template <typename A> __device__ __forceinline__ bool is_nan(A v) {
  if constexpr (std::is_floating_point<A>::value) return v != v;
  else return false;
}
// Every reduction also names what happens to an element as it is loaded (pre) and to the finished value as it
// is stored (post); `factor` is the reduction's one parameter (1 / count for the mean, the exponent p for a
// p-norm).  The plain reductions load unchanged and store through project().
struct RNoTransform {
  template <typename A> static __device__ __forceinline__ A pre(A v, float) { return v; }
  template <typename A> static __device__ __forceinline__ A post(A v, float factor, int is_mean) {
    return project<A>(v, factor, is_mean);
  }
};
struct RSum : RNoTransform {
  template <typename A> static __device__ __forceinline__ A identity() { return A(0); }
  template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a + b; }
};
// p-norms: sum |x|^p, stored as its p-th root (Norm1.cu:17-56); p = 1 and p = 2 without a pow()
template <typename A> __device__ __forceinline__ A abs_of(A v) { return v < A(0) ? -v : v; }
struct RNorm1 : RSum {
  template <typename A> static __device__ __forceinline__ A pre(A v, float) { return abs_of(v); }
  template <typename A> static __device__ __forceinline__ A post(A v, float, int) { return v; }
};
struct RNorm2 : RSum {
  template <typename A> static __device__ __forceinline__ A pre(A v, float) { return v * v; }
  template <typename A> static __device__ __forceinline__ A post(A v, float, int) {
    if constexpr (std::is_same<A, double>::value) return sqrt(v);
    else return A(sqrtf(float(v)));
  }
};
struct RNormP : RSum {
  template <typename A> static __device__ __forceinline__ A pre(A v, float p) {
    if constexpr (std::is_same<A, double>::value) return pow(abs_of(v), double(p));
    else return A(powf(float(abs_of(v)), p));
  }
  template <typename A> static __device__ __forceinline__ A post(A v, float p, int) {
    if constexpr (std::is_same<A, double>::value) return pow(v, 1.0 / double(p));
    else return A(powf(float(v), 1.0f / p));
  }
};
struct RProd : RNoTransform {
  template <typename A> static __device__ __forceinline__ A identity() { return A(1); }
  template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a * b; }
};
struct RMax : RNoTransform {
  template <typename A> static __device__ __forceinline__ A identity() {
    if constexpr (std::is_floating_point<A>::value) return -std::numeric_limits<A>::infinity();
    else return std::numeric_limits<A>::lowest();
  }
  template <typename A> static __device__ __forceinline__ A apply(A a, A b) {
    // fp32: the hardware's NaN-propagating maximum (one v_maximum3_f32)
    if constexpr (std::is_same<A, float>::value) return __builtin_elementwise_maximum(a, b);
    else return (is_nan(a) || a > b) ? a : (is_nan(b) ? b : (a > b ? a : b));
  }
};
struct RMin : RNoTransform {
  template <typename A> static __device__ __forceinline__ A identity() {
    if constexpr (std::is_floating_point<A>::value) return std::numeric_limits<A>::infinity();
    else return std::numeric_limits<A>::max();
  }
  template <typename A> static __device__ __forceinline__ A apply(A a, A b) {
    if constexpr (std::is_same<A, float>::value) return __builtin_elementwise_minimum(a, b);
    else return (is_nan(a) || a < b) ? a : (is_nan(b) ? b : (a < b ? a : b));
  }
};
// R without its load transform: what folds partial results, which went through pre() when they were formed
template <typename R> struct Folded : R {
  template <typename A> static __device__ __forceinline__ A pre(A v, float) { return v; }
};
// the float face the wave / block reduction helpers expect
template <typename R> struct AsFloatOp {
  static __device__ __forceinline__ float identity() { return R::template identity<float>(); }
  static __device__ __forceinline__ float apply(float a, float b) { return R::template apply<float>(a, b); }
};

template <typename R, typename ACC>
__device__ __forceinline__ ACC block_reduce_lds(ACC v, ACC* lds) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
    if (tid < s) lds[tid] = R::template apply<ACC>(lds[tid], lds[tid + s]);
    __syncthreads();
  }
  ACC r = lds[0];
  __syncthreads();
  return r;
}

// ---------------------------------------------------------------------------
// inner reduction, vector path (fp32 / bf16 / fp16 input, fp32 accumulate)
// grid = (row groups, nsplit); a group of `tpr` threads takes one row chunk
// ---------------------------------------------------------------------------
struct InnerArgs {
  const void* in;
  void* out;          // OUT_T [rows] when nsplit == 1, else float [rows, nsplit]
  int64_t rows;
  int64_t row_stride; // elements
  int64_t cols;
  int64_t chunk;      // columns per split (multiple of the vector width)
  int nsplit;
  float factor;
  int is_mean;
};

template <typename T, typename OUT_T, bool WAVE_ROW, typename R>
__global__ __launch_bounds__(WAVE_ROW ? 256 : 1024)
void reduce_inner_vec_kernel(InnerArgs a) {
  constexpr int VEC = VecIO<T>::N;
  constexpr int U = 8;
  __shared__ float red[kMaxWaves];
  const int tpr = WAVE_ROW ? kWave : int(blockDim.x);
  const int t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  const int64_t row = WAVE_ROW
      ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index()
      : int64_t(blockIdx.x);
  if (WAVE_ROW && row >= a.rows) return;
  const int split = blockIdx.y;
  const int64_t c0 = int64_t(split) * a.chunk;
  const int64_t c1 = (c0 + a.chunk < a.cols) ? c0 + a.chunk : a.cols;
  const T* p = static_cast<const T*>(a.in) + row * a.row_stride + c0;
  const int64_t nvec = (c1 - c0) / VEC;

  float acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) acc[u] = R::template identity<float>();
  int64_t v = t;
  for (; v + int64_t(U - 1) * tpr < nvec; v += int64_t(U) * tpr) {
    u32x4 r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) r[u] = ld16(p + (v + int64_t(u) * tpr) * VEC);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float f[VEC];
      VecIO<T>::unpack(r[u], f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[u] = R::apply(acc[u], R::pre(f[j], a.factor));
    }
  }
  for (; v < nvec; v += tpr) {
    float f[VEC];
    VecIO<T>::unpack(ld16(p + v * VEC), f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[0] = R::apply(acc[0], R::pre(f[j], a.factor));
  }
  // scalar tail of the last split
  for (int64_t c = c0 + nvec * VEC + t; c < c1; c += tpr)
    acc[1] = R::apply(acc[1], R::pre(Cvt<T>::load(static_cast<const T*>(a.in) + row * a.row_stride + c), a.factor));
  float s = R::apply(R::apply(R::apply(acc[0], acc[1]), R::apply(acc[2], acc[3])),
                     R::apply(R::apply(acc[4], acc[5]), R::apply(acc[6], acc[7])));
  if constexpr (WAVE_ROW) {
    s = wave_allreduce<AsFloatOp<R>>(s);
  } else {
    s = block_allreduce<AsFloatOp<R>>(s, red, int(blockDim.x >> 6));
  }
  if (t == 0) {
    if (a.nsplit == 1) st_acc<OUT_T, float>(static_cast<OUT_T*>(a.out) + row, R::template post<float>(s, a.factor, a.is_mean));
    else static_cast<float*>(a.out)[row * a.nsplit + split] = s;
  }
}

// inner reduction, scalar path: any dtype / alignment; one workgroup per row
template <typename T, typename ACC, typename OUT_T, typename R>
__global__ __launch_bounds__(256)
void reduce_inner_scalar_kernel(const T* in, OUT_T* out, int64_t rows, int64_t row_stride,
                                int64_t cols, float factor, int is_mean) {
  __shared__ ACC lds[256];
  const int64_t row = blockIdx.x;
  const T* p = in + row * row_stride;
  ACC acc = R::template identity<ACC>();
  for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) acc = R::template apply<ACC>(acc, R::template pre<ACC>(ld_acc<T, ACC>(p + c), factor));
  acc = block_reduce_lds<R, ACC>(acc, lds);
  if (threadIdx.x == 0) st_acc<OUT_T, ACC>(out + row, R::template post<ACC>(acc, factor, is_mean));
}

// ---------------------------------------------------------------------------
// outer reduction, vector path: in [B, R, C] (C unit stride), out [B, C]
// grid = (column tiles of 64 vectors, row splits, B); block = 64 x WY
// ---------------------------------------------------------------------------
struct OuterArgs {
  const void* in;
  void* out;            // OUT_T [B, C] when rsplit == 1, else float [rsplit, B, C]
  int64_t B, R, C;
  int64_t b_stride, r_stride;   // elements
  int64_t rows_per_split;
  int rsplit;
  int wx;               // wavefronts of a workgroup side by side across columns (the others stack over rows)
  float factor;
  int is_mean;
  int split_major;      // grid = (row splits, column tiles, batch) instead of (column tiles, row splits, batch)
};

template <typename T, typename OUT_T, typename R>
__global__ __launch_bounds__(512)
void reduce_outer_vec_kernel(OuterArgs a) {
  constexpr int VEC = VecIO<T>::N;
  constexpr int U = 8;
  extern __shared__ float lds[];   // [WY][WX][VEC][64]
  const int lane = threadIdx.x & 63;
  const int wave = wave_index();
  const int wx = a.wx;
  const int wc = wave % wx;        // this wavefront's place across columns ...
  const int w = wave / wx;         // ... and over rows
  const int wy = int(blockDim.x >> 6) / wx;
  // Row splits along the grid's x (whenever the column tiles fit its y): workgroups are dealt to the XCDs round
  // robin in x-major order, so the workgroups of one XCD then take whole runs of rows (every column tile of a few
  // row splits) rather than one column tile of every row split -- the same bytes in flight at any time, 1 % faster
  // (32768 x 4096 bf16: 42.5 against 42.9 us, both orders measured alternately)
  const int split = a.split_major ? blockIdx.x : blockIdx.y;
  const int64_t tile = a.split_major ? blockIdx.y : blockIdx.x;
  const int64_t cv = (tile * wx + wc) * kWave + lane;   // column vector index
  const int64_t c = cv * VEC;
  const bool col_ok = c < a.C;                              // C is a multiple of VEC here
  const int64_t b = blockIdx.z;
  const int64_t r0 = int64_t(split) * a.rows_per_split;
  const int64_t r1 = (r0 + a.rows_per_split < a.R) ? r0 + a.rows_per_split : a.R;
  const T* p = static_cast<const T*>(a.in) + b * a.b_stride + c;

  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc[j] = R::template identity<float>();
  if (col_ok) {
    // a wavefront takes U consecutive rows per step, the workgroup wy * U consecutive rows: measured faster than
    // interleaving the wavefronts row by row (41.0 against 42.3 us at 32768 x 4096 bf16)
    int64_t r = r0 + int64_t(w) * U;
    for (; r + U <= r1; r += int64_t(U) * wy) {
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = ld16(p + (r + u) * a.r_stride);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float f[VEC];
        VecIO<T>::unpack(v[u], f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = R::apply(acc[j], R::pre(f[j], a.factor));
      }
    }
    // the last, partial run of rows of this wavefront (fewer than U)
    for (; r < r1; ++r) {
      float f[VEC];
      VecIO<T>::unpack(ld16(p + r * a.r_stride), f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = R::apply(acc[j], R::pre(f[j], a.factor));
    }
  }
  // fold the waves of the block: lane-major layout keeps LDS accesses conflict-free
#pragma unroll
  for (int j = 0; j < VEC; ++j) lds[((w * wx + wc) * VEC + j) * kWave + lane] = acc[j];
  __syncthreads();
  // thread (w, lane) finishes element j = w, w + wy, ... of its lane's vector
  for (int j = w; j < VEC; j += wy) {
    float s = R::template identity<float>();
    for (int k = 0; k < wy; ++k) s = R::apply(s, lds[((k * wx + wc) * VEC + j) * kWave + lane]);
    if (col_ok) {
      if (a.rsplit == 1)
        st_acc<OUT_T, float>(static_cast<OUT_T*>(a.out) + b * a.C + c + j, R::template post<float>(s, a.factor, a.is_mean));
      else
        static_cast<float*>(a.out)[(int64_t(split) * a.B + b) * a.C + c + j] = s;
    }
  }
}

// folds float partials [nparts, n] -> OUT_T [n]
template <typename OUT_T, typename R>
__global__ __launch_bounds__(256)
void reduce_fold_partials_kernel(const float* part, OUT_T* out, int nparts, int64_t n, float factor,
                                 int is_mean) {
  // 64 outputs per block; the 4 waves take interleaved partial rows with 8
  // independent loads in flight each, then fold through LDS
  constexpr int U = 8;
  __shared__ float lds[4][kWave];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t i = int64_t(blockIdx.x) * kWave + lane;
  float acc = R::template identity<float>();
  if (i < n) {
    int k = w;
    for (; k + (U - 1) * 4 < nparts; k += U * 4) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = part[int64_t(k + u * 4) * n + i];
#pragma unroll
      for (int u = 0; u < U; ++u) acc = R::apply(acc, v[u]);
    }
    for (; k < nparts; k += 4) acc = R::apply(acc, part[int64_t(k) * n + i]);
  }
  lds[w][lane] = acc;
  __syncthreads();
  if (w == 0 && i < n) {
    const float s = R::apply(R::apply(lds[0][lane], lds[1][lane]), R::apply(lds[2][lane], lds[3][lane]));
    st_acc<OUT_T, float>(out + i, R::template post<float>(s, factor, is_mean));
  }
}

// outer reduction, scalar path: one thread per output column, any dtype
template <typename T, typename ACC, typename OUT_T, typename R>
__global__ __launch_bounds__(256)
void reduce_outer_scalar_kernel(const T* in, OUT_T* out, int64_t B, int64_t NR, int64_t C,
                                int64_t b_stride, int64_t r_stride, float factor, int is_mean) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= B * C) return;
  const int64_t b = i / C, c = i - b * C;
  const T* p = in + b * b_stride + c;
  ACC acc = R::template identity<ACC>();
  for (int64_t r = 0; r < NR; ++r) acc = R::template apply<ACC>(acc, R::template pre<ACC>(ld_acc<T, ACC>(p + r * r_stride), factor));
  st_acc<OUT_T, ACC>(out + i, R::template post<ACC>(acc, factor, is_mean));
}

// ---------------------------------------------------------------------------
// generic strided reduction: one thread per output element
// ---------------------------------------------------------------------------
constexpr int kMaxDims = 8;
struct GenericMeta {
  int n_keep, n_red;
  int64_t keep_size[kMaxDims], keep_stride[kMaxDims];   // outermost first
  int64_t red_size[kMaxDims], red_stride[kMaxDims];     // outermost first
  int64_t n_out, n_red_total;
};

template <typename T, typename ACC, typename OUT_T, typename R>
__global__ __launch_bounds__(256)
void reduce_generic_kernel(const T* in, OUT_T* out, GenericMeta m, float factor, int is_mean) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= m.n_out) return;
  int64_t rem = i, base = 0;
  for (int d = m.n_keep - 1; d >= 0; --d) {
    const int64_t q = rem / m.keep_size[d];
    base += (rem - q * m.keep_size[d]) * m.keep_stride[d];
    rem = q;
  }
  ACC acc = R::template identity<ACC>();
  for (int64_t k = 0; k < m.n_red_total; ++k) {
    int64_t r = k, off = base;
    for (int d = m.n_red - 1; d >= 0; --d) {
      const int64_t q = r / m.red_size[d];
      off += (r - q * m.red_size[d]) * m.red_stride[d];
      r = q;
    }
    acc = R::template apply<ACC>(acc, R::template pre<ACC>(ld_acc<T, ACC>(in + off), factor));
  }
  st_acc<OUT_T, ACC>(out + i, R::template post<ACC>(acc, factor, is_mean));
}

// ---------------------------------------------------------------------------
// host-side planning
// ---------------------------------------------------------------------------
struct MergedDim { int64_t size, stride; bool reduce; };

enum PlanKind { PLAN_EMPTY, PLAN_COPYLIKE, PLAN_INNER, PLAN_OUTER, PLAN_GENERIC };

struct ReducePlan {
  PlanKind kind = PLAN_GENERIC;
  std::vector<MergedDim> dims;     // outermost first, extents > 1 only
  int64_t n_out = 1, n_red = 1;
  // inner
  int64_t rows = 1, row_stride = 0, cols = 1;
  // outer
  int64_t B = 1, R = 1, C = 1, b_stride = 0, r_stride = 0;
};

// Same merging rule as the reference planner: walk from the innermost
// dimension outwards and fuse a dimension into its inner neighbour when both
// are reduced or both are kept and stride[i] == stride[i+1] * shape[i+1].
static int make_plan(int ndim, const int64_t* shape, const int64_t* strides, int naxes,
                     const int64_t* axes, ReducePlan* plan, const char* who) {
  HK_REQUIRE(ndim >= 0 && ndim <= kMaxDims, HK_ERR_INVALID, "%s: ndim %d not in [0, %d]", who, ndim, kMaxDims);
  HK_REQUIRE(naxes >= 0, HK_ERR_INVALID, "%s: negative axis count", who);
  HK_REQUIRE(ndim == 0 || (shape && strides), HK_ERR_INVALID, "%s: null shape/strides", who);
  HK_REQUIRE(naxes == 0 || axes, HK_ERR_INVALID, "%s: null axes", who);
  bool red[kMaxDims] = {false};
  for (int i = 0; i < naxes; ++i) {
    HK_REQUIRE(axes[i] >= 0 && axes[i] < ndim, HK_ERR_INVALID, "%s: axis %lld out of range for %d dims",
               who, (long long)axes[i], ndim);
    red[axes[i]] = true;     // duplicates collapse, order is irrelevant
  }
  plan->dims.clear();
  plan->n_out = 1;
  plan->n_red = 1;
  for (int d = 0; d < ndim; ++d) {
    HK_REQUIRE(shape[d] >= 0, HK_ERR_INVALID, "%s: negative extent", who);
    if (red[d]) plan->n_red *= shape[d]; else plan->n_out *= shape[d];
  }
  if (plan->n_out == 0) { plan->kind = PLAN_EMPTY; return HK_OK; }
  std::vector<MergedDim> rev;   // innermost first
  for (int d = ndim - 1; d >= 0; --d) {
    if (shape[d] == 1) continue;
    if (!rev.empty() && rev.back().reduce == red[d] &&
        strides[d] == rev.back().stride * rev.back().size) {
      rev.back().size *= shape[d];
    } else {
      rev.push_back(MergedDim{shape[d], strides[d], red[d]});
    }
  }
  plan->dims.assign(rev.rbegin(), rev.rend());
  std::vector<MergedDim> keep, rd;
  for (auto& d : plan->dims) (d.reduce ? rd : keep).push_back(d);
  if (rd.empty() || plan->n_red == 1) {
    plan->kind = PLAN_COPYLIKE;   // nothing to add up: generic kernel copies / scales
    return HK_OK;
  }
  if (plan->n_red == 0) { plan->kind = PLAN_GENERIC; return HK_OK; }  // sum over nothing = 0
  const auto& dims = plan->dims;
  if (rd.size() == 1 && rd[0].stride == 1 && keep.size() <= 1) {
    plan->kind = PLAN_INNER;
    plan->cols = rd[0].size;
    plan->rows = keep.empty() ? 1 : keep[0].size;
    plan->row_stride = keep.empty() ? 0 : keep[0].stride;
    return HK_OK;
  }
  if (rd.size() == 1 && !dims.back().reduce && dims.back().stride == 1 && keep.size() <= 2 &&
      dims.size() >= 2 && dims[dims.size() - 2].reduce) {
    plan->kind = PLAN_OUTER;
    plan->C = dims.back().size;
    plan->R = rd[0].size;
    plan->r_stride = rd[0].stride;
    plan->B = keep.size() == 2 ? keep[0].size : 1;
    plan->b_stride = keep.size() == 2 ? keep[0].stride : 0;
    return HK_OK;
  }
  plan->kind = PLAN_GENERIC;
  return HK_OK;
}

struct InnerShape { int tpr; int nsplit; int64_t chunk; bool vec; };
struct OuterShape { int wy; int wx; int rsplit; int64_t rows_per_split; bool vec; };

template <typename T>
static InnerShape shape_inner(const ReducePlan& p, const void* in) {
  constexpr int VEC = 16 / sizeof(T);
  InnerShape s{};
  s.vec = aligned16(in) && (p.rows == 1 || p.row_stride % VEC == 0);
  const int64_t nvec = p.cols / VEC;
  int tpr = tune_get(TUNE_REDUCE_INNER_THREADS);
  const int64_t want_blocks = int64_t(device_cu_count()) * 4;
  if (tpr <= 0) {
    tpr = nvec <= 64 * 32 ? 64 : (nvec <= 256 * 32 ? 256 : 1024);
    // too few rows to fill the chip: widen the group until a thread has at most one round of 8 loads,
    // so that a short row costs one memory round trip instead of several dependent ones
    if (p.rows < want_blocks) tpr = int(std::max<int64_t>(tpr, std::min<int64_t>(1024, (nvec + 7) / 8)));
  }
  tpr = std::min(1024, std::max(64, (tpr + 63) / 64 * 64));
  s.tpr = tpr;
  // few long rows: split columns so that ~4 workgroups per CU exist
  int64_t groups = tpr == 64 ? (p.rows + 3) / 4 : p.rows;
  int64_t nsplit = 1;
  if (groups < want_blocks && nvec > int64_t(tpr) * 32) {
    nsplit = std::min<int64_t>((want_blocks + groups - 1) / groups, nvec / (int64_t(tpr) * 16));
    nsplit = std::max<int64_t>(1, std::min<int64_t>(nsplit, 1024));
  }
  int64_t chunk_vec = (nvec + nsplit - 1) / nsplit;
  if (chunk_vec == 0) chunk_vec = 1;
  s.chunk = chunk_vec * VEC;
  s.nsplit = int((p.cols + s.chunk - 1) / s.chunk);
  if (s.nsplit < 1) s.nsplit = 1;
  return s;
}

template <typename T>
static OuterShape shape_outer(const ReducePlan& p, const void* in) {
  constexpr int VEC = 16 / sizeof(T);
  OuterShape s{};
  s.vec = aligned16(in) && p.C % VEC == 0 && p.r_stride % VEC == 0 && (p.B == 1 || p.b_stride % VEC == 0);
  s.wy = 1; s.wx = 1; s.rsplit = 1; s.rows_per_split = p.R;
  if (!s.vec) return s;
  int64_t col_tiles = std::max<int64_t>(1, (p.C / VEC + 63) / 64);
  // waves per block: enough rows per wave to keep 8 loads in flight
  // Measured at 32768 x 4096 bf16 (whole call, one workgroup per compute unit): 4 wavefronts 42.5 us, 8 wavefronts
  // 43.4 us, 16 wavefronts 44.3 us; putting 2, 4 or 8 of them side by side across columns (a workgroup then reads
  // 2 KiB or more of consecutive bytes per row) changed nothing (43.2 .. 43.5 us), so the default keeps one.
  int waves = tune_get(TUNE_REDUCE_OUTER_WAVES) > 0 ? std::min(8, tune_get(TUNE_REDUCE_OUTER_WAVES)) : 4;
  int wx = tune_get(TUNE_REDUCE_OUTER_WAVES_ACROSS) > 0 ? tune_get(TUNE_REDUCE_OUTER_WAVES_ACROSS) : 1;
  while (wx > 1 && (wx > waves || col_tiles % wx != 0)) wx >>= 1;
  int wy = waves / wx;
  while (wy > 1 && p.R < int64_t(wy) * 8) wy >>= 1;
  s.wy = wy;
  s.wx = wx;
  col_tiles /= wx;
  int rsplit = tune_get(TUNE_REDUCE_OUTER_ROW_BLOCKS);
  if (rsplit <= 0) {
    const int64_t want_blocks = int64_t(device_cu_count());   // one workgroup per CU measured fastest
    const int64_t have = col_tiles * p.B;
    rsplit = int(std::max<int64_t>(1, (want_blocks + have - 1) / have));
  }
  const int64_t max_split = std::max<int64_t>(1, p.R / (int64_t(wy) * 8));
  rsplit = int(std::min<int64_t>(rsplit, max_split));
  rsplit = std::min(rsplit, 65535);
  s.rows_per_split = (p.R + rsplit - 1) / rsplit;
  s.rsplit = int((p.R + s.rows_per_split - 1) / s.rows_per_split);
  return s;
}

template <typename T>
static size_t workspace_for(const ReducePlan& p, const void* in) {
  if (p.kind == PLAN_INNER) {
    InnerShape s = shape_inner<T>(p, in);
    return (s.vec && s.nsplit > 1) ? size_t(p.rows) * s.nsplit * sizeof(float) : 0;
  }
  if (p.kind == PLAN_OUTER) {
    OuterShape s = shape_outer<T>(p, in);
    return (s.vec && s.rsplit > 1) ? size_t(s.rsplit) * p.B * p.C * sizeof(float) : 0;
  }
  return 0;
}

static GenericMeta generic_meta(const ReducePlan& p) {
  GenericMeta m{};
  m.n_keep = 0; m.n_red = 0;
  for (auto& d : p.dims) {
    if (d.reduce) { m.red_size[m.n_red] = d.size; m.red_stride[m.n_red] = d.stride; ++m.n_red; }
    else { m.keep_size[m.n_keep] = d.size; m.keep_stride[m.n_keep] = d.stride; ++m.n_keep; }
  }
  m.n_out = p.n_out;
  m.n_red_total = p.n_red;
  return m;
}

// fast kernels: T in {float, bf16, fp16}, fp32 accumulation
template <typename T, typename OUT_T, typename R>
static int reduce_fast(const ReducePlan& p, const void* in, void* out, float factor, int is_mean,
                       void* ws, size_t ws_bytes, hipStream_t st, bool* handled) {
  *handled = false;
  if (p.kind == PLAN_INNER) {
    InnerShape s = shape_inner<T>(p, in);
    if (!s.vec) return HK_OK;
    *handled = true;
    InnerArgs a{};
    a.in = in; a.rows = p.rows; a.row_stride = p.row_stride; a.cols = p.cols; a.chunk = s.chunk;
    a.nsplit = s.nsplit; a.factor = factor; a.is_mean = is_mean;
    if (s.nsplit > 1) {
      const size_t need = size_t(p.rows) * s.nsplit * sizeof(float);
      HK_REQUIRE(ws && ws_bytes >= need, HK_ERR_WORKSPACE, "hk_reduce: workspace of %zu bytes needed, %zu given", need, ws_bytes);
      a.out = ws;
    } else {
      a.out = out;
    }
    HK_REQUIRE(p.rows <= 0x7fffffffLL, HK_ERR_INVALID, "hk_reduce: too many rows");
    profile_before(st);
    if (s.tpr == 64) {
      dim3 grid(unsigned((p.rows + 3) / 4), unsigned(s.nsplit)), block(256);
      HK_LAUNCH((reduce_inner_vec_kernel<T, OUT_T, true, R>), grid, block, 0, st, a);
    } else {
      dim3 grid(unsigned(p.rows), unsigned(s.nsplit)), block{unsigned(s.tpr)};
      HK_LAUNCH((reduce_inner_vec_kernel<T, OUT_T, false, R>), grid, block, 0, st, a);
    }
    profile_after(st);
    int rc = launch_check("reduce_inner_vec_kernel");
    if (rc != HK_OK || s.nsplit == 1) return rc;
    // second pass over the fp32 partials [rows, nsplit]: combine and store only, the elements' own
    // transform (|x|, x^2, |x|^p of the p-norms) was applied when the partials were formed
    HK_LAUNCH((reduce_inner_scalar_kernel<float, float, OUT_T, Folded<R>>), dim3(unsigned(p.rows)), dim3(256), 0, st,
                       static_cast<const float*>(ws), static_cast<OUT_T*>(out), p.rows, int64_t(s.nsplit),
                       int64_t(s.nsplit), factor, is_mean);
    return launch_check("reduce_inner_scalar_kernel");
  }
  if (p.kind == PLAN_OUTER) {
    OuterShape s = shape_outer<T>(p, in);
    if (!s.vec) return HK_OK;
    *handled = true;
    constexpr int VEC = 16 / sizeof(T);
    OuterArgs a{};
    a.in = in; a.B = p.B; a.R = p.R; a.C = p.C; a.b_stride = p.b_stride; a.r_stride = p.r_stride;
    a.rows_per_split = s.rows_per_split; a.rsplit = s.rsplit; a.wx = s.wx; a.factor = factor; a.is_mean = is_mean;
    if (s.rsplit > 1) {
      const size_t need = size_t(s.rsplit) * p.B * p.C * sizeof(float);
      HK_REQUIRE(ws && ws_bytes >= need, HK_ERR_WORKSPACE, "hk_reduce: workspace of %zu bytes needed, %zu given", need, ws_bytes);
      a.out = ws;
    } else {
      a.out = out;
    }
    HK_REQUIRE(p.B <= 65535, HK_ERR_UNSUPPORTED, "hk_reduce: batch extent %lld too large for the column kernel", (long long)p.B);
    const int64_t col_tiles = ((p.C / VEC + 63) / 64 + s.wx - 1) / s.wx;
    a.split_major = col_tiles <= 65535 ? 1 : 0;
    dim3 grid(unsigned(col_tiles), unsigned(s.rsplit), unsigned(p.B)), block{unsigned(64 * s.wy * s.wx)};
    if (a.split_major) grid = dim3(unsigned(s.rsplit), unsigned(col_tiles), unsigned(p.B));
    const size_t lds = size_t(s.wy) * s.wx * 64 * VEC * sizeof(float);
    profile_before(st);
    HK_LAUNCH((reduce_outer_vec_kernel<T, OUT_T, R>), grid, block, lds, st, a);
    profile_after(st);
    int rc = launch_check("reduce_outer_vec_kernel");
    if (rc != HK_OK || s.rsplit == 1) return rc;
    const int64_t n = p.B * p.C;
    HK_LAUNCH((reduce_fold_partials_kernel<OUT_T, R>), dim3(unsigned((n + 63) / 64)), dim3(256), 0, st,
                       static_cast<const float*>(ws), static_cast<OUT_T*>(out), s.rsplit, n, factor, is_mean);
    return launch_check("reduce_fold_partials_kernel");
  }
  return HK_OK;
}

template <typename T, typename ACC, typename OUT_T, typename R>
static int reduce_slow(const ReducePlan& p, const void* in, void* out, float factor, int is_mean,
                       hipStream_t st) {
  const T* ip = static_cast<const T*>(in);
  OUT_T* op = static_cast<OUT_T*>(out);
  if (p.kind == PLAN_INNER) {
    HK_REQUIRE(p.rows <= 0x7fffffffLL, HK_ERR_INVALID, "hk_reduce: too many rows");
    HK_LAUNCH((reduce_inner_scalar_kernel<T, ACC, OUT_T, R>), dim3(unsigned(p.rows)), dim3(256), 0, st, ip, op,
                       p.rows, p.row_stride, p.cols, factor, is_mean);
    return launch_check("reduce_inner_scalar_kernel");
  }
  if (p.kind == PLAN_OUTER) {
    const int64_t n = p.B * p.C;
    HK_LAUNCH((reduce_outer_scalar_kernel<T, ACC, OUT_T, R>), dim3(unsigned((n + 255) / 256)), dim3(256), 0, st,
                       ip, op, p.B, p.R, p.C, p.b_stride, p.r_stride, factor, is_mean);
    return launch_check("reduce_outer_scalar_kernel");
  }
  GenericMeta m = generic_meta(p);
  HK_LAUNCH((reduce_generic_kernel<T, ACC, OUT_T, R>), dim3(unsigned((m.n_out + 255) / 256)), dim3(256), 0, st,
                     ip, op, m, factor, is_mean);
  return launch_check("reduce_generic_kernel");
}

template <typename T, typename OUT_T, typename R>
static int reduce_float_like(const ReducePlan& p, const void* in, void* out, float factor, int is_mean,
                             void* ws, size_t ws_bytes, hipStream_t st) {
  bool handled = false;
  int rc = reduce_fast<T, OUT_T, R>(p, in, out, factor, is_mean, ws, ws_bytes, st, &handled);
  if (rc != HK_OK || handled) return rc;
  return reduce_slow<T, float, OUT_T, R>(p, in, out, factor, is_mean, st);
}

// every dtype of one reduction
template <typename R>
static int reduce_typed(const ReducePlan& q, int in_dtype, int out_dtype, const void* in, void* out, float factor,
                        int is_mean, void* workspace, size_t workspace_bytes, hipStream_t st) {
#define HK_RED_SLOW(T) return reduce_slow<T, AccOf<T>::type, T, R>(q, in, out, factor, is_mean, st)
  switch (in_dtype) {
    case HK_FLOAT32: return reduce_float_like<float, float, R>(q, in, out, factor, is_mean, workspace, workspace_bytes, st);
    case HK_BFLOAT16:
      if (out_dtype == HK_FLOAT32) return reduce_float_like<bf16, float, R>(q, in, out, factor, is_mean, workspace, workspace_bytes, st);
      return reduce_float_like<bf16, bf16, R>(q, in, out, factor, is_mean, workspace, workspace_bytes, st);
    case HK_FLOAT16:
      if (out_dtype == HK_FLOAT32) return reduce_float_like<fp16, float, R>(q, in, out, factor, is_mean, workspace, workspace_bytes, st);
      return reduce_float_like<fp16, fp16, R>(q, in, out, factor, is_mean, workspace, workspace_bytes, st);
    case HK_FLOAT64: HK_RED_SLOW(double);
    case HK_UINT8: HK_RED_SLOW(uint8_t);
    case HK_INT8: HK_RED_SLOW(int8_t);
    case HK_INT16: HK_RED_SLOW(int16_t);
    case HK_INT32: HK_RED_SLOW(int32_t);
    case HK_INT64: HK_RED_SLOW(int64_t);
    default:
      set_last_error("hk_reduce: not implemented for dtype %d", in_dtype);
      return HK_ERR_UNSUPPORTED;
  }
#undef HK_RED_SLOW
}

// p-norm over one dimension: floating types only
template <typename R>
static int norm_typed(const ReducePlan& q, int dtype, const void* in, void* out, float p, void* workspace,
                      size_t workspace_bytes, hipStream_t st) {
  switch (dtype) {
    case HK_FLOAT32: return reduce_float_like<float, float, R>(q, in, out, p, 0, workspace, workspace_bytes, st);
    case HK_BFLOAT16: return reduce_float_like<bf16, bf16, R>(q, in, out, p, 0, workspace, workspace_bytes, st);
    case HK_FLOAT16: return reduce_float_like<fp16, fp16, R>(q, in, out, p, 0, workspace, workspace_bytes, st);
    case HK_FLOAT64: return reduce_slow<double, double, double, R>(q, in, out, p, 0, st);
    default:
      set_last_error("hk_norm: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

// Gradient of the p-norm over the middle dimension of a dense [before, reduce, after] array
// (norm_gradient_kernel, Norm1.cu:59-97): with n = the norm and g = its gradient of the slice,
//   p = 1: sign(x) * g;   p = 2: g * x / n;   p > 2: x * |x|^(p-2) * g / n^(p-1);   0 where n == 0.
template <typename T, typename CT>
__global__ __launch_bounds__(256)
void norm_grad_kernel(const T* __restrict__ x, const T* __restrict__ norm, const T* __restrict__ grad, T* out,
                      int64_t total, int64_t reduce_size, int64_t after, int64_t p) {
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t b = i / (reduce_size * after);
  const int64_t a = i % after;
  const int64_t y = b * after + a;
  const CT xv = CT(Cvt<T>::load(x + i)), g = CT(Cvt<T>::load(grad + y));
  CT o;
  if (p == 1) {
    o = (xv == CT(0) ? CT(0) : (xv < CT(0) ? CT(-1) : CT(1))) * g;
  } else {
    const CT n = CT(Cvt<T>::load(norm + y));
    if (n == CT(0)) o = CT(0);
    else if (p == 2) o = g * xv / n;
    else o = xv * CT(pow(double(abs_of(xv)), double(p - 2))) * g / CT(pow(double(n), double(p - 1)));
  }
  Cvt<T>::store(out + i, o);
}

// the same for a norm over the last dimension (after == 1), one 16-byte vector per thread.  PK names the
// exponent at compile time (1, 2, or 0 for any other) so that nothing but the arithmetic sits between the loads
// and the store; the per-row factor is formed once per thread.
template <typename T, int PK>
__global__ __launch_bounds__(kStreamThreads)
void norm_grad_rows_vec_kernel(const T* __restrict__ x, const T* __restrict__ norm, const T* __restrict__ grad,
                               T* out, uint32_t nvec, uint32_t cols_vec, int64_t p) {
  constexpr int VEC = VecIO<T>::N;
  const uint32_t v = blockIdx.x * uint32_t(kStreamThreads) + threadIdx.x;
  if (v >= nvec) return;
  const uint32_t r = v / cols_vec;
  const u32x4 raw = ld16(x + size_t(v) * VEC);
  const float g = Cvt<T>::load(grad + r);
  const float n = PK == 1 ? 1.f : Cvt<T>::load(norm + r);
  float f[VEC];
  VecIO<T>::unpack(raw, f);
  if constexpr (PK == 1) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = (f[j] == 0.f ? 0.f : (f[j] < 0.f ? -1.f : 1.f)) * g;
  } else if constexpr (PK == 2) {
    const float scale = n == 0.f ? 0.f : g / n;
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = n == 0.f ? 0.f : f[j] * scale;
  } else {
    const float scale = n == 0.f ? 0.f : g / powf(n, float(p - 1));
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = n == 0.f ? 0.f : f[j] * powf(fabsf(f[j]), float(p - 2)) * scale;
  }
  st16_stream(out + size_t(v) * VEC, VecIO<T>::pack(f));
}

template <typename T>
static int norm_grad_typed(const void* x, const void* norm, const void* grad, void* out, int64_t before,
                           int64_t reduce_size, int64_t after, int64_t p, hipStream_t s) {
  const int64_t total = before * reduce_size * after;
  using CT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  if constexpr (!std::is_same<T, double>::value) {
    constexpr int VEC = VecIO<T>::N;
    if (after == 1 && reduce_size % VEC == 0 && aligned16(x) && aligned16(out) && total / VEC < 0x7fffffffLL) {
      const uint32_t nvec = uint32_t(total / VEC);
      auto kernel = p == 1 ? norm_grad_rows_vec_kernel<T, 1>
                  : p == 2 ? norm_grad_rows_vec_kernel<T, 2> : norm_grad_rows_vec_kernel<T, 0>;
      profile_before(s);
      HK_LAUNCH(kernel, dim3((nvec + kStreamThreads - 1) / kStreamThreads), dim3(kStreamThreads), 0, s,
                         static_cast<const T*>(x), static_cast<const T*>(norm), static_cast<const T*>(grad),
                         static_cast<T*>(out), nvec, uint32_t(reduce_size / VEC), p);
      profile_after(s);
      return launch_check("norm_grad_rows_vec_kernel");
    }
  }
  HK_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_norm_bwd: array too large");
  profile_before(s);
  HK_LAUNCH((norm_grad_kernel<T, CT>), dim3(unsigned((total + 255) / 256)), dim3(256), 0, s,
                     static_cast<const T*>(x), static_cast<const T*>(norm), static_cast<const T*>(grad),
                     static_cast<T*>(out), total, reduce_size, after, p);
  profile_after(s);
  return launch_check("norm_grad_kernel");
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_norm(int dtype, const void* in, void* out, int ndim, const int64_t* shape, const int64_t* strides,
            int64_t dim, int64_t p, void* workspace, size_t workspace_bytes, hkStream_t stream) {
  HK_REQUIRE(p >= 1, HK_ERR_INVALID, "hk_norm: p must be at least 1, got %lld", (long long) p);
  HK_REQUIRE(dim >= 0 && dim < ndim, HK_ERR_INVALID, "hk_norm: dim %lld outside [0, %d)", (long long) dim, ndim);
  ReducePlan q;
  int rc = make_plan(ndim, shape, strides, 1, &dim, &q, "hk_norm");
  if (rc != HK_OK) return rc;
  if (q.kind == PLAN_EMPTY) return HK_OK;
  HK_REQUIRE(out, HK_ERR_INVALID, "hk_norm: null output");
  HK_REQUIRE(in || q.n_red == 0, HK_ERR_INVALID, "hk_norm: null input");
  HK_REQUIRE((q.n_out + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_norm: output too large");
  if (q.kind == PLAN_COPYLIKE || q.n_red == 0) q.kind = PLAN_GENERIC;   // extent 0 or 1: one thread per output
  hipStream_t st = as_hip(stream);
  if (p == 1) return norm_typed<RNorm1>(q, dtype, in, out, 1.f, workspace, workspace_bytes, st);
  if (p == 2) return norm_typed<RNorm2>(q, dtype, in, out, 2.f, workspace, workspace_bytes, st);
  return norm_typed<RNormP>(q, dtype, in, out, float(p), workspace, workspace_bytes, st);
}

int hk_norm_bwd(int dtype, const void* in, const void* norm, const void* grad, void* out, int64_t before,
                int64_t reduce_size, int64_t after, int64_t p, hkStream_t stream) {
  HK_REQUIRE(p >= 1, HK_ERR_INVALID, "hk_norm_bwd: p must be at least 1, got %lld", (long long) p);
  HK_REQUIRE(before >= 0 && reduce_size >= 0 && after >= 0, HK_ERR_INVALID, "hk_norm_bwd: negative shape");
  if (before == 0 || reduce_size == 0 || after == 0) return HK_OK;
  HK_REQUIRE(in && grad && out && (norm || p == 1), HK_ERR_INVALID, "hk_norm_bwd: null input/output");
  hipStream_t s = as_hip(stream);
  switch (dtype) {
    case HK_FLOAT32: return norm_grad_typed<float>(in, norm, grad, out, before, reduce_size, after, p, s);
    case HK_BFLOAT16: return norm_grad_typed<bf16>(in, norm, grad, out, before, reduce_size, after, p, s);
    case HK_FLOAT16: return norm_grad_typed<fp16>(in, norm, grad, out, before, reduce_size, after, p, s);
    case HK_FLOAT64: return norm_grad_typed<double>(in, norm, grad, out, before, reduce_size, after, p, s);
    default:
      set_last_error("hk_norm_bwd: not implemented for dtype %d", dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

int hk_reduce_workspace_bytes(int in_dtype, int ndim, const int64_t* shape, const int64_t* strides,
                              int naxes, const int64_t* axes, size_t* bytes) {
  HK_REQUIRE(bytes, HK_ERR_INVALID, "hk_reduce_workspace_bytes: null output");
  *bytes = 0;
  ReducePlan p;
  int rc = make_plan(ndim, shape, strides, naxes, axes, &p, "hk_reduce_workspace_bytes");
  if (rc != HK_OK) return rc;
  // alignment of the data pointer is unknown here: assume the vector path
  const void* aligned = reinterpret_cast<const void*>(uintptr_t(16));
  switch (in_dtype) {
    case HK_FLOAT32: *bytes = workspace_for<float>(p, aligned); break;
    case HK_BFLOAT16: case HK_FLOAT16: *bytes = workspace_for<uint16_t>(p, aligned); break;
    default: break;
  }
  return HK_OK;
}

int hk_reduce(int in_dtype, int out_dtype, const void* in, void* out, int ndim, const int64_t* shape,
              const int64_t* strides, int naxes, const int64_t* axes, int op, void* workspace,
              size_t workspace_bytes, hkStream_t stream) {
  HK_REQUIRE(op == HK_REDUCE_SUM || op == HK_REDUCE_MEAN || op == HK_REDUCE_MAX || op == HK_REDUCE_MIN ||
             op == HK_REDUCE_PROD, HK_ERR_UNSUPPORTED, "hk_reduce: reduction %d not implemented", op);
  ReducePlan p;
  int rc = make_plan(ndim, shape, strides, naxes, axes, &p, "hk_reduce");
  if (rc != HK_OK) return rc;
  if (p.kind == PLAN_EMPTY) return HK_OK;   // nothing to write
  HK_REQUIRE(out, HK_ERR_INVALID, "hk_reduce: null output");
  if (naxes == 0) {   // nothing to reduce: the dense copy of the input
    HK_REQUIRE(out_dtype == in_dtype, HK_ERR_UNSUPPORTED, "hk_reduce: a reduction over no axes cannot change the dtype");
    return hk_strided_copy(in_dtype, in, out, ndim, shape, strides, stream);
  }
  const bool additive = op == HK_REDUCE_SUM || op == HK_REDUCE_MEAN;
  if (p.n_red == 0 && additive) {
    // empty sums are 0; an empty mean is 0 * (1/0) = NaN for floating types (all-ones bytes are a NaN in each)
    const bool floating = out_dtype == HK_FLOAT16 || out_dtype == HK_BFLOAT16 || out_dtype == HK_FLOAT32 || out_dtype == HK_FLOAT64;
    const size_t es = dtype_size(out_dtype);
    HK_REQUIRE(es > 0, HK_ERR_UNSUPPORTED, "hk_reduce: dtype %d not implemented", out_dtype);
    return hk_memset(out, (op == HK_REDUCE_MEAN && floating) ? 0xFF : 0, size_t(p.n_out) * es, stream);
  }
  HK_REQUIRE(in || p.n_red == 0, HK_ERR_INVALID, "hk_reduce: null input");
  HK_REQUIRE((p.n_out + 255) / 256 <= 0x7fffffffLL, HK_ERR_INVALID, "hk_reduce: output too large");
  const int is_mean = op == HK_REDUCE_MEAN;
  const float factor = is_mean ? 1.0f / float(size_t(p.n_red)) : 1.0f;
  hipStream_t st = as_hip(stream);
  const bool in16 = in_dtype == HK_BFLOAT16 || in_dtype == HK_FLOAT16;
  // a wider output exists for sums and products of 16-bit data (ReduceSum.cu:28-37, ReduceProd.cu:26-37)
  const bool widen_ok = in16 && out_dtype == HK_FLOAT32 && op != HK_REDUCE_MAX && op != HK_REDUCE_MIN;
  HK_REQUIRE(out_dtype == in_dtype || widen_ok, HK_ERR_UNSUPPORTED,
             "hk_reduce: output dtype %d not implemented for input dtype %d and reduction %d", out_dtype, in_dtype, op);
  ReducePlan q = p;
  // an empty reduced extent (max / min / prod) writes the identity: the one-thread-per-output kernel does that
  if (p.kind == PLAN_COPYLIKE || p.n_red == 0) q.kind = PLAN_GENERIC;
  switch (op) {
    case HK_REDUCE_MAX: return reduce_typed<RMax>(q, in_dtype, out_dtype, in, out, factor, 0, workspace, workspace_bytes, st);
    case HK_REDUCE_MIN: return reduce_typed<RMin>(q, in_dtype, out_dtype, in, out, factor, 0, workspace, workspace_bytes, st);
    case HK_REDUCE_PROD: return reduce_typed<RProd>(q, in_dtype, out_dtype, in, out, factor, 0, workspace, workspace_bytes, st);
    default: return reduce_typed<RSum>(q, in_dtype, out_dtype, in, out, factor, is_mean, workspace, workspace_bytes, st);
  }
}

} // extern "C"
