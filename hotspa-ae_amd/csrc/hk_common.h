// Device-side building blocks shared by every row-wise kernel: 128-bit vector
// I/O for fp32 / bf16 / fp16 rows, wave64 DPP reductions, LDS cross-wave
// combine, and the host-side launch/error helpers of the C-ABI layer.
//
// Written for gfx950 (CDNA4) only: wave size is 64, DPP row_bcast modes and the
// v_cvt_pk_bf16_f32 conversion are assumed.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <type_traits>
#include <utility>
#include <stdint.h>
#include <stddef.h>

#include "hk_rowwise.h"

namespace hk {

constexpr int kWave = 64;
constexpr int kMaxBlock = 1024;
constexpr int kMaxWaves = kMaxBlock / kWave;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Storage element tags. bf16 / fp16 are carried as raw 16-bit patterns; all
// arithmetic is done in fp32 after unpacking.
struct bf16 { uint16_t bits; };
struct fp16 { uint16_t bits; };

// Index of the calling wavefront inside its workgroup as a scalar: everything
// derived from it (row number, row pointers) then lives in SGPRs and row loads
// use one scalar base plus a per-lane offset.
__device__ __forceinline__ int wave_index() {
  return __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6));
}

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---------------------------------------------------------------------------
// Scalar conversions
// ---------------------------------------------------------------------------
template <typename T> struct Cvt;

template <> struct Cvt<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ float to_float(float v) { return v; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};

template <> struct Cvt<bf16> {
  static __device__ __forceinline__ float load(const bf16* p) {
    return u2f(uint32_t(p->bits) << 16);
  }
  static __device__ __forceinline__ float to_float(bf16 v) { return u2f(uint32_t(v.bits) << 16); }
  static __device__ __forceinline__ void store(bf16* p, float v) {
    // round-to-nearest-even through the hardware packed converter
    f32x2 f = {v, 0.f};
    bf16x2 b = __builtin_convertvector(f, bf16x2);
    p->bits = uint16_t(__builtin_bit_cast(uint32_t, b) & 0xffffu);
  }
};

template <> struct Cvt<fp16> {
  static __device__ __forceinline__ float load(const fp16* p) {
    return float(__builtin_bit_cast(_Float16, p->bits));
  }
  static __device__ __forceinline__ float to_float(fp16 v) { return float(__builtin_bit_cast(_Float16, v.bits)); }
  static __device__ __forceinline__ void store(fp16* p, float v) {
    p->bits = __builtin_bit_cast(uint16_t, _Float16(v));
  }
};

template <> struct Cvt<double> {
  static __device__ __forceinline__ double load(const double* p) { return *p; }
  static __device__ __forceinline__ void store(double* p, double v) { *p = v; }
};

// ---------------------------------------------------------------------------
// 16-byte vectors: N elements of T <-> N floats
// ---------------------------------------------------------------------------
template <typename T> struct VecIO;

template <> struct VecIO<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    f[0] = u2f(r.x); f[1] = u2f(r.y); f[2] = u2f(r.z); f[3] = u2f(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 r = {f2u(f[0]), f2u(f[1]), f2u(f[2]), f2u(f[3])};
    return r;
  }
};

template <> struct VecIO<bf16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    f[0] = u2f(r.x << 16); f[1] = u2f(r.x & 0xffff0000u);
    f[2] = u2f(r.y << 16); f[3] = u2f(r.y & 0xffff0000u);
    f[4] = u2f(r.z << 16); f[5] = u2f(r.z & 0xffff0000u);
    f[6] = u2f(r.w << 16); f[7] = u2f(r.w & 0xffff0000u);
  }
  static __device__ __forceinline__ uint32_t pk(float a, float b) {
    f32x2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 r = {pk(f[0], f[1]), pk(f[2], f[3]), pk(f[4], f[5]), pk(f[6], f[7])};
    return r;
  }
};

template <> struct VecIO<fp16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void up(uint32_t w, float* f) {
    f32x2 v = __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
    f[0] = v.x; f[1] = v.y;
  }
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    up(r.x, f); up(r.y, f + 2); up(r.z, f + 4); up(r.w, f + 6);
  }
  static __device__ __forceinline__ uint32_t pk(float a, float b) {
    f32x2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 r = {pk(f[0], f[1]), pk(f[2], f[3]), pk(f[4], f[5]), pk(f[6], f[7])};
    return r;
  }
};

// max(a, b, c) in one instruction.  Written as inline assembly because fmaxf() on values that were
// assembled from integer bits makes the compiler canonicalise each operand first (one extra v_max per
// element); the instruction itself already returns the non-NaN operand when one operand is a NaN.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// A 16-byte vector whose every element is -infinity in T: padding that leaves a
// maximum and a sum of exponentials untouched, so kernels need no per-vector
// predicate in their arithmetic.
template <typename T> __device__ __forceinline__ u32x4 neg_inf_vec();
template <> __device__ __forceinline__ u32x4 neg_inf_vec<float>() {
  return u32x4{0xff800000u, 0xff800000u, 0xff800000u, 0xff800000u};
}
template <> __device__ __forceinline__ u32x4 neg_inf_vec<bf16>() {
  return u32x4{0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u};
}
template <> __device__ __forceinline__ u32x4 neg_inf_vec<fp16>() {
  return u32x4{0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u};
}

// Row data is read exactly once: non-temporal loads keep it from displacing
// reusable lines and stream measurably faster.  Small reused vectors (gamma,
// beta) go through ld16_keep.
__device__ __forceinline__ u32x4 ld16(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ u32x4 ld16_keep(const void* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ void st16(void* p, const u32x4& v) {
  *reinterpret_cast<u32x4*>(p) = v;
}
// Streaming store for write-once outputs (bypasses cache residency).
__device__ __forceinline__ void st16_stream(void* p, const u32x4& v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
// Buffer addressing: a 128-bit resource descriptor (base address + byte count) held in scalar registers, plus a
// per-lane byte offset.  The hardware checks every lane's offset against the byte count: a load past the end
// returns zeros and a store past the end is dropped, so a kernel that walks a row in whole vectors needs no branch
// around its memory instructions for a ragged last step.  One descriptor addresses at most 4 GiB.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
// Workgroup size of the kernels that read an array and write an array with no step across threads (element-wise
// operators, gradients formed from a stored row statistic): one wavefront, one 16-byte vector per thread.  Measured
// on 1 GiB bf16 arrays, exp(x): 64 threads 311 us, 64 x 2 vectors 317 us, 128 x 2 318 us, 256 threads 319 us,
// 512 threads 332 us; the plain copy of the streaming yardstick orders the shapes the same way.  Write-only
// kernels (fills, broadcasts) stay at 256 threads, where that stream is fastest.
constexpr int kStreamThreads = 64;

constexpr int kBufKeep = 0;     // default cache policy (reused data: gamma, beta)
constexpr int kBufStream = 2;   // "nt": data touched once (rows in, rows out)
__device__ __forceinline__ BufferRsrc make_rsrc(const void* base, uint32_t bytes) {
  // word 3 = 0x00020000: raw buffer, 32-bit data format, no swizzle (the gfx9 / CDNA encoding)
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, int(bytes), 0x00020000);
}
template <int POLICY>
__device__ __forceinline__ u32x4 buf_ld16(BufferRsrc r, uint32_t byte_offset) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, int(byte_offset), 0, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void buf_st16(BufferRsrc r, uint32_t byte_offset, const u32x4& v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, int(byte_offset), 0, POLICY);
}

__device__ __forceinline__ u32x4 ld16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

// Rows on up to three levels.  The leading dimensions of a row-major operand need not step by one constant
// pitch: a view with permuted leading dimensions (x.permute(0, 2, 1, 3) of a [B, H, S, D] array) numbers its rows
// r = (i2 * c1 + i1) * c0 + i0 and row r starts i0 * s0 + i1 * s1 + i2 * s2 elements from the base, the three
// steps being whatever the view's strides are.  A dense or row-pitched array is the one-level case.
//
// A launch WALKS the levels in an order of its own choosing (plan_row_walk below puts the level with the smallest
// steps first, so that neighbouring workgroups touch neighbouring memory whatever the view's own order is): walk
// index (j0, j1, j2), j_k < n_k, is the row whose operands start j0 * pitch + j1 * p1 + j2 * p2 elements from their
// bases (the operand's steps in walk order) and whose NUMBER, the index into the dense [rows] arrays next to the
// operands (statistics, labels, losses), is j0 * rn0 + j1 * rn1 + j2 * rn2.  The one-shot row kernels get the
// decomposition for nothing: they run on a three-dimensional grid whose x walks j0 and whose y / z are j1 / j2.
// One level is n = {rows, 1, 1}, rn = {1, 0, 0}.
struct LevelSteps {
  int64_t p1, p2;   // elements between consecutive j1 / j2; the step of j0 is the operand's pitch
};
struct RowNumbering {
  int64_t rn0, rn1, rn2;
};
// offset of this workgroup's rows along the two outer walk levels, in elements
__device__ __forceinline__ int64_t outer_level_offset(const LevelSteps& l) {
  return int64_t(blockIdx.y) * l.p1 + int64_t(blockIdx.z) * l.p2;
}
// number of the row (j0, blockIdx.y, blockIdx.z)
__device__ __forceinline__ int64_t dense_row_index(int64_t j0, const RowNumbering& rn) {
  return j0 * rn.rn0 + int64_t(blockIdx.y) * rn.rn1 + int64_t(blockIdx.z) * rn.rn2;
}
// (j0, j1, j2) of walk index r, for kernels that walk the rows themselves
struct RowSplit {
  uint32_t j0, j1, j2;
};
__device__ __forceinline__ RowSplit split_row(int64_t r, int64_t n0, int64_t n1) {
  RowSplit s;
  const uint32_t q = uint32_t(r) / uint32_t(n0);
  s.j0 = uint32_t(r) - q * uint32_t(n0);
  s.j2 = q / uint32_t(n1);
  s.j1 = q - s.j2 * uint32_t(n1);
  return s;
}
__device__ __forceinline__ int64_t split_offset(const RowSplit& s, int64_t pitch, const LevelSteps& l) {
  return int64_t(s.j0) * pitch + int64_t(s.j1) * l.p1 + int64_t(s.j2) * l.p2;
}
__device__ __forceinline__ int64_t split_number(const RowSplit& s, const RowNumbering& rn) {
  return int64_t(s.j0) * rn.rn0 + int64_t(s.j1) * rn.rn1 + int64_t(s.j2) * rn.rn2;
}

// ---------------------------------------------------------------------------
// wave64 reductions through DPP (no LDS traffic).  After the call every lane
// holds the result.
// ---------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float v, float old = 0.f) {
  return u2f(uint32_t(__builtin_amdgcn_update_dpp(
      int(f2u(old)), int(f2u(v)), CTRL, ROW_MASK, 0xf, false)));
}

// The four controls below permute the lanes of a row of 16 among themselves: every lane has a source, so the
// "old" operand never shows.  Passing 0 with bound_ctrl set lets the compiler fold the move into the instruction
// that consumes it (one v_add_f32 with a DPP operand instead of copy + v_mov_b32_dpp + add).
template <int CTRL>
__device__ __forceinline__ float dpp_perm(float v) {
  return u2f(uint32_t(__builtin_amdgcn_update_dpp(0, int(f2u(v)), CTRL, 0xf, 0xf, true)));
}

constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror
constexpr int kDppMirror = 0x140;     // row_mirror
constexpr int kDppBcast15 = 0x142;    // row_bcast:15
constexpr int kDppBcast31 = 0x143;    // row_bcast:31

__device__ __forceinline__ float readlane_f(float v, int lane) {
  return u2f(uint32_t(__builtin_amdgcn_readlane(int(f2u(v)), lane)));
}

// Op: a struct with `static float identity()` and `static float apply(float, float)`.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v) {
  v = Op::apply(v, dpp_perm<kDppXor1>(v));
  v = Op::apply(v, dpp_perm<kDppXor2>(v));
  v = Op::apply(v, dpp_perm<kDppHalfMirror>(v));
  v = Op::apply(v, dpp_perm<kDppMirror>(v));
  // every lane of a 16-lane row now holds that row's result; fold the 4 rows
  float r0 = readlane_f(v, 0), r1 = readlane_f(v, 16);
  float r2 = readlane_f(v, 32), r3 = readlane_f(v, 48);
  return Op::apply(Op::apply(r0, r1), Op::apply(r2, r3));
}


// Shuffle through DPP for the 16-lane-local steps of a butterfly, and through
// the cross-lane network only for the 16 / 32 strides.  Used by reductions on
// tuples (Chan merge, online softmax) where the combine is not a plain op.
template <int STRIDE>
__device__ __forceinline__ float lane_xor(float v) {
  if constexpr (STRIDE == 1) return dpp_perm<kDppXor1>(v);
  else if constexpr (STRIDE == 2) return dpp_perm<kDppXor2>(v);
  else return __shfl_xor(v, STRIDE, kWave);
}

// ---------------------------------------------------------------------------
// Block-level combine: waves [w0, w0+nw) of a workgroup cooperate on one row.
// `scratch` holds kMaxWaves floats per slot in LDS.  All threads of the block
// must call (contains __syncthreads).
// ---------------------------------------------------------------------------
template <typename Op>
__device__ __forceinline__ float block_allreduce(float v, float* scratch, int nwaves) {
  v = wave_allreduce<Op>(v);
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) scratch[w] = v;
  __syncthreads();
  float r = Op::identity();
  for (int i = 0; i < nwaves; ++i) r = Op::apply(r, scratch[i]);
  return r;
}

// ---------------------------------------------------------------------------
// Tuple reductions.  P is a struct with `float v[P::K]` and
// `static P merge(P, P)` (commutative up to rounding).  The wave version
// leaves the same value in every lane; the group version combines the waves
// [first_wave, first_wave + nwaves) of a workgroup through `scratch`
// (kMaxWaves * K floats) and contains one __syncthreads().
// ---------------------------------------------------------------------------
template <typename P>
__device__ __forceinline__ P wave_allreduce_tuple(P a) {
  P b;
#pragma unroll
  for (int k = 0; k < P::K; ++k) b.v[k] = dpp_perm<kDppXor1>(a.v[k]);
  a = P::merge(a, b);
#pragma unroll
  for (int k = 0; k < P::K; ++k) b.v[k] = dpp_perm<kDppXor2>(a.v[k]);
  a = P::merge(a, b);
#pragma unroll
  for (int k = 0; k < P::K; ++k) b.v[k] = dpp_perm<kDppHalfMirror>(a.v[k]);
  a = P::merge(a, b);
#pragma unroll
  for (int k = 0; k < P::K; ++k) b.v[k] = dpp_perm<kDppMirror>(a.v[k]);
  a = P::merge(a, b);
  P r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int k = 0; k < P::K; ++k) r[j].v[k] = readlane_f(a.v[k], 16 * j);
  return P::merge(P::merge(r[0], r[1]), P::merge(r[2], r[3]));
}

// the cross-wave half of group_allreduce_tuple: `a` is already the same in every lane of a wave
template <typename P>
__device__ __forceinline__ P group_combine_tuple(P a, float* scratch, int first_wave, int nwaves);

template <typename P>
__device__ __forceinline__ P group_allreduce_tuple(P a, float* scratch, int first_wave,
                                                    int nwaves) {
  a = wave_allreduce_tuple<P>(a);
  return group_combine_tuple<P>(a, scratch, first_wave, nwaves);
}

// Every thread walks the group's waves in order.  The reads are wave-uniform LDS broadcasts which the
// compiler keeps in flight together; a butterfly over per-lane reads (one LDS round trip, then DPP merges on
// every lane) was measured slower at every group width (5120-column LayerNorm backward, ten waves: 96.5
// against 91.0 us).
template <typename P>
__device__ __forceinline__ P group_combine_tuple(P a, float* scratch, int first_wave, int nwaves) {
  if (nwaves == 1) return a;
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < P::K; ++k) scratch[w * P::K + k] = a.v[k];
  }
  __syncthreads();
  P r;
#pragma unroll
  for (int k = 0; k < P::K; ++k) r.v[k] = scratch[first_wave * P::K + k];
  for (int i = 1; i < nwaves; ++i) {
    P o;
#pragma unroll
    for (int k = 0; k < P::K; ++k) o.v[k] = scratch[(first_wave + i) * P::K + k];
    r = P::merge(r, o);
  }
  return r;
}

// The same for a group that is the whole workgroup and whose number of wavefronts is a constant: no loop, the
// NW partials are read with wide LDS loads at constant offsets.
template <typename P, int NW>
__device__ __forceinline__ P group_allreduce_tuple_fixed(P a, float* scratch) {
  a = wave_allreduce_tuple<P>(a);
  if constexpr (NW == 1) return a;
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < P::K; ++k) scratch[w * P::K + k] = a.v[k];
  }
  __syncthreads();
  P r;
#pragma unroll
  for (int k = 0; k < P::K; ++k) r.v[k] = scratch[k];
#pragma unroll
  for (int i = 1; i < NW; ++i) {
    P o;
#pragma unroll
    for (int k = 0; k < P::K; ++k) o.v[k] = scratch[i * P::K + k];
    r = P::merge(r, o);
  }
  return r;
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index is a
// compile-time constant in every iteration
template <typename F, int... D>
__device__ __forceinline__ void static_for_impl(F& f, std::integer_sequence<int, D...>) {
  (f(std::integral_constant<int, D>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// plain sums of K values
template <int KK>
struct SumTuple {
  static constexpr int K = KK;
  float v[KK];
  static __device__ __forceinline__ SumTuple identity() {
    SumTuple r;
#pragma unroll
    for (int k = 0; k < KK; ++k) r.v[k] = 0.f;
    return r;
  }
  static __device__ __forceinline__ SumTuple merge(SumTuple a, const SumTuple& b) {
#pragma unroll
    for (int k = 0; k < KK; ++k) a.v[k] += b.v[k];
    return a;
  }
};

// (count, mean, M2) with Chan's parallel update of Welford's statistics
struct MomentTuple {
  static constexpr int K = 3;
  float v[3];
  static __device__ __forceinline__ MomentTuple identity() { return MomentTuple{{0.f, 0.f, 0.f}}; }
  static __device__ __forceinline__ MomentTuple merge(const MomentTuple& a, const MomentTuple& b) {
    MomentTuple r;
    const float n = a.v[0] + b.v[0];
    const float inv = n > 0.f ? __builtin_amdgcn_rcpf(n) : 0.f;
    const float delta = b.v[1] - a.v[1];
    const float wb = b.v[0] * inv;
    r.v[0] = n;
    r.v[1] = a.v[1] + delta * wb;
    r.v[2] = a.v[2] + b.v[2] + delta * delta * a.v[0] * wb;
    return r;
  }
};

// The same update when both sides are known to hold the SAME number of elements (every step of a
// butterfly over lanes that started with equal counts): the weights are 1/2, no reciprocal is needed.
struct EqualMomentTuple {
  static constexpr int K = 3;
  float v[3];
  static __device__ __forceinline__ EqualMomentTuple merge(const EqualMomentTuple& a, const EqualMomentTuple& b) {
    EqualMomentTuple r;
    const float delta = b.v[1] - a.v[1];
    r.v[0] = a.v[0] + a.v[0];
    r.v[1] = fmaf(delta, 0.5f, a.v[1]);
    r.v[2] = fmaf(delta * delta, 0.5f * a.v[0], a.v[2] + b.v[2]);
    return r;
  }
};

// Online softmax state.  v[0] = ml, the running maximum ALREADY multiplied by
// log2(e) and rounded to fp32 once; v[1] = sum of exp2(x * log2e - ml).  Every
// exponential of a thread is taken against the thread's own rounded ml and
// re-based by exp2(ml_a - ml_b), a difference of two fp32 numbers, so the
// rounding of ml is a common factor of numerator and denominator and cancels:
// results do not degrade when the logits carry a large common offset.
// K3 variant: v[2] additionally tracks the maximum itself (for log-sum-exp).
template <int KK>
struct OnlineSoftmaxTuple {
  static constexpr int K = KK;
  float v[KK];
  static __device__ __forceinline__ OnlineSoftmaxTuple identity() {
    OnlineSoftmaxTuple r;
    r.v[0] = -__builtin_huge_valf();
    r.v[1] = 0.f;
    if constexpr (KK == 3) r.v[2] = -__builtin_huge_valf();
    return r;
  }
  static __device__ __forceinline__ OnlineSoftmaxTuple merge(const OnlineSoftmaxTuple& a,
                                                              const OnlineSoftmaxTuple& b) {
    OnlineSoftmaxTuple r;
    const float m = fmaxf(a.v[0], b.v[0]);
    // an empty side has ml = -inf and sum = 0; keep exp2(-inf - -inf) out of the result
    const float ms = (m == -__builtin_huge_valf()) ? 0.f : m;
    r.v[0] = m;
    r.v[1] = a.v[1] * __builtin_amdgcn_exp2f(a.v[0] - ms) + b.v[1] * __builtin_amdgcn_exp2f(b.v[0] - ms);
    if constexpr (KK == 3) r.v[2] = fmaxf(a.v[2], b.v[2]);
    return r;
  }
};
using MaxSumTuple = OnlineSoftmaxTuple<2>;
using MaxSumMaxTuple = OnlineSoftmaxTuple<3>;

// ---------------------------------------------------------------------------
// host helpers
// ---------------------------------------------------------------------------
void set_last_error(const char* fmt, ...);

#define HK_CHECK_HIP(expr)                                                     \
  do {                                                                         \
    hipError_t _e = (expr);                                                    \
    if (_e != hipSuccess) {                                                    \
      ::hk::set_last_error("%s failed: %s (%s:%d)", #expr,                     \
                           hipGetErrorString(_e), __FILE__, __LINE__);         \
      return HK_ERR_HIP;                                                       \
    }                                                                          \
  } while (0)

#define HK_REQUIRE(cond, code, ...)                                            \
  do {                                                                         \
    if (!(cond)) {                                                             \
      ::hk::set_last_error(__VA_ARGS__);                                       \
      return (code);                                                           \
    }                                                                          \
  } while (0)

// The constant enters the arithmetic rounded to the array's type, as static_cast<spec_t>(value) does.
template <typename T> inline double round_const(double c) { return c; }
template <> inline double round_const<float>(double c) { return double(float(c)); }
template <> inline double round_const<fp16>(double c) { return double(float(_Float16(float(c)))); }
template <> inline double round_const<bf16>(double c) {
  const float f = float(c);
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return c;          // NaN stays NaN
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;     // round to nearest even
  float r;
  __builtin_memcpy(&r, &u, 4);
  return double(r);
}

inline double round_to_dtype(int dtype, double c) {
  switch (dtype) {
    case HK_FLOAT32: return round_const<float>(c);
    case HK_BFLOAT16: return round_const<bf16>(c);
    case HK_FLOAT16: return round_const<fp16>(c);
    default: return c;
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The order in which a launch walks the levels of its rows (see LevelSteps).  level_rows = the counts in the
// rows' own numbering (innermost first); key = per level, the sum of the operands' steps.  Levels are taken by
// ascending key, levels of a single row last.  on_grid: the walk rides on a grid (x = walk level 0 carries up to
// four rows per workgroup, y / z hold at most 65535): level 0 is then the first level in that order with at least
// eight rows, if there is one; an order whose y / z do not fit gives way to the rows' own order, then to the
// longest level on x.  The caller checks n[1], n[2] against the grid's limits (walk_fits_grid).  perm[k] = the level
// walked k-th.
struct RowWalk {
  int perm[3];
  int64_t n[3];
  RowNumbering rn;
};
inline RowWalk plan_row_walk(const int64_t level_rows[3], const int64_t key[3], bool on_grid) {
  int order[3] = {0, 1, 2};
  auto before = [&](int a, int b) {
    const bool ea = level_rows[a] == 1, eb = level_rows[b] == 1;
    if (ea != eb) return eb;
    if (key[a] != key[b]) return key[a] < key[b];
    return a < b;
  };
  for (int i = 0; i < 3; ++i)
    for (int j = i + 1; j < 3; ++j)
      if (before(order[j], order[i])) { const int t = order[i]; order[i] = order[j]; order[j] = t; }
  if (on_grid) {
    int first = -1;
    for (int k = 0; k < 3 && first < 0; ++k)
      if (level_rows[order[k]] >= 8) first = k;
    if (first > 0) {
      const int lead = order[first];
      for (int k = first; k > 0; --k) order[k] = order[k - 1];
      order[0] = lead;
    }
    auto fits = [&] { return level_rows[order[1]] <= 65535 && level_rows[order[2]] <= 65535; };
    if (!fits()) { order[0] = 0; order[1] = 1; order[2] = 2; }
    if (!fits()) {
      int longest = 0;
      for (int k = 1; k < 3; ++k)
        if (level_rows[k] > level_rows[longest]) longest = k;
      order[0] = longest; order[1] = longest == 0 ? 1 : 0; order[2] = longest == 2 ? 1 : 2;
    }
  }
  const int64_t number[3] = {1, level_rows[0], level_rows[0] * level_rows[1]};
  RowWalk w;
  for (int k = 0; k < 3; ++k) { w.perm[k] = order[k]; w.n[k] = level_rows[order[k]]; }
  w.rn = RowNumbering{number[order[0]], number[order[1]], number[order[2]]};
  return w;
}
inline bool walk_fits_grid(const RowWalk& w) { return w.n[0] <= 0x7fffffffLL && w.n[1] <= 65535 && w.n[2] <= 65535; }
// an operand's steps in walk order
inline void walk_steps(const RowWalk& w, const int64_t steps[3], int64_t* pitch, LevelSteps* lv) {
  *pitch = steps[w.perm[0]];
  lv->p1 = steps[w.perm[1]];
  lv->p2 = steps[w.perm[2]];
}

inline hipStream_t as_hip(hkStream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Tunable launch parameters (0 = automatic); values are set through
// hk_tune_set().  The order matches the name table in hk_device.hip.
enum TuneKey {
  TUNE_NORM_FWD_THREADS = 0,
  TUNE_NORM_BWD_THREADS,
  TUNE_NORM_BWD_BLOCKS,
  TUNE_SOFTMAX_THREADS,
  TUNE_SCE_THREADS,
  TUNE_REDUCE_INNER_THREADS,
  TUNE_REDUCE_OUTER_ROW_BLOCKS,
  TUNE_NORM_BWD_ROWS_PER_BLOCK,
  TUNE_NORM_BWD_PREFETCH,
  TUNE_REDUCE_OUTER_WAVES_ACROSS,
  TUNE_REDUCE_OUTER_WAVES,
  TUNE_NORM_FWD_ROWS,
  TUNE_NORM_FWD_RESIDENT,
  TUNE_NUM_KEYS
};
int tune_get(int key);
int device_cu_count();
void device_lds_bytes(size_t* per_cu, size_t* per_block);

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case HK_UINT8: case HK_INT8: case HK_BOOL: return 1;
    case HK_INT16: case HK_FLOAT16: case HK_BFLOAT16: return 2;
    case HK_INT32: case HK_FLOAT32: return 4;
    case HK_INT64: case HK_FLOAT64: return 8;
    default: return 0;
  }
}

int launch_check(const char* what);

// Timing of an operator's main kernel with the events armed through hk_profile_next_kernel().  profile_before()
// hands the armed pair to the next HK_LAUNCH made by this thread, which binds both events to that very dispatch
// (hipExtLaunchKernelGGL): their difference is the kernel's own begin-to-end time, as a kernel trace reports it,
// without the few microseconds between an event marker on the stream and the kernel's start.  profile_after()
// drops a pair that no launch took (an early error return).  All three are no-ops when nothing is armed.
void profile_before(hipStream_t s);
void profile_after(hipStream_t s);
bool profile_claim(hipEvent_t* before, hipEvent_t* after);

// Dynamic LDS to ask for so that at most `workgroups` workgroups of a kernel are resident on a compute unit
// (`static_bytes` = the kernel's own __shared__ arrays; the compute unit's LDS as the device reports it): half way
// between the size that would let one more in and the size that would keep one out, so the allocation granule does
// not matter.  A streaming kernel whose threads hold several vectors in flight moves more with fewer workgroups
// per compute unit than the thread limit allows (RMSNorm forward, 256-thread workgroups: 8 resident 84.8 us, 5
// resident 83.5 us).  Returns false when one workgroup may not ask for that much (a residency the device cannot be
// held to this way).
static inline bool lds_bytes_for_residency(int workgroups, size_t static_bytes, size_t* bytes) {
  *bytes = 0;
  if (workgroups <= 0) return true;
  size_t total = 0, per_block = 0;
  device_lds_bytes(&total, &per_block);
  const size_t want = (total / size_t(workgroups + 1) + total / size_t(workgroups)) / 2;
  if (want > per_block) return false;
  *bytes = want > static_bytes ? want - static_bytes : 0;
  return true;
}

#define HK_LAUNCH(kernel, grid, block, lds_bytes, stream, ...)                                                  \
  do {                                                                                                          \
    hipEvent_t hk_ev_before_, hk_ev_after_;                                                                     \
    if (::hk::profile_claim(&hk_ev_before_, &hk_ev_after_))                                                     \
      hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, hk_ev_before_, hk_ev_after_, 0, __VA_ARGS__); \
    else                                                                                                        \
      hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, __VA_ARGS__);                                  \
  } while (0)

} // namespace hk
