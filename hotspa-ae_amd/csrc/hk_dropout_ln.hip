// Dropout-add-LayerNorm / RMSNorm with every feature of the interface: dropout,
// per-row and per-column scaling, row subsets, mixed input / residual / weight
// types and the parallel-residual form.  Calls that use none of these are handed
// to the plain norm kernels; this file is the general path.
//
// Work split: a thread owns chunks of 8 consecutive columns (one 16-byte vector
// of a 16-bit type, two of fp32).  Forward: one group of threads per row, the row
// in registers, statistics as in the plain kernel (Welford / Chan for LayerNorm,
// two sums for RMSNorm).  Backward: a persistent grid of column-owner groups
// keeps up to five per-column sums in registers and writes one fp32 partial row
// per group; a second kernel folds the partial rows.
//
// Dropout mask: element e of the input draws word e % 4 of Philox4x32-10 (key =
// seed, counter = (2 * (e / 4) + input number, offset)), so the mask does not
// depend on the launch shape.
#include "hk_common.h"

#include <algorithm>
#include <type_traits>

namespace hk {

// ---------------------------------------------------------------------------
// Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11)
// ---------------------------------------------------------------------------
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                              uint32_t k0, uint32_t k1, uint32_t out[4]) {
  constexpr uint32_t kM0 = 0xD2511F53u, kM1 = 0xCD9E8D57u, kW0 = 0x9E3779B9u, kW1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = uint64_t(kM0) * c0;
    const uint64_t p1 = uint64_t(kM1) * c2;
    const uint32_t n0 = uint32_t(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = uint32_t(p0 >> 32) ^ c3 ^ k1;
    c1 = uint32_t(p1);
    c3 = uint32_t(p0);
    c0 = n0;
    c2 = n2;
    k0 += kW0;
    k1 += kW1;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

struct DropArgs {
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  float keep_p;
};

// Keep bits of the 8 elements [e0, e0 + 8) of input number `which` (e0 is a multiple of 8): bit j set =
// element e0 + j is kept.  A draw is float(bits) * 2^-32 + 2^-33 in (0, 1], kept when <= keep_p.
__device__ __forceinline__ uint32_t keep_bits8(int64_t e0, int which, const DropArgs& d) {
  const uint64_t g2 = (uint64_t(e0) >> 1) + uint64_t(which);   // 2 * (e0 / 4) + which
  uint32_t bits = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint64_t g = g2 + uint64_t(2 * h);
    uint32_t r[4];
    philox4x32_10(uint32_t(g), uint32_t(g >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi, r);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float u = fmaf(float(r[j]), 2.3283064365386963e-10f, 1.1641532182693481e-10f);
      bits |= (u <= d.keep_p ? 1u : 0u) << (4 * h + j);
    }
  }
  return bits;
}

// 8 mask bytes (0 / 1) as one 8-byte store / load
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_mask8(uint8_t* p, uint32_t bits) {
  uint32_t w0 = 0, w1 = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    w0 |= ((bits >> j) & 1u) << (8 * j);
    w1 |= ((bits >> (4 + j)) & 1u) << (8 * j);
  }
  *reinterpret_cast<u32x2*>(p) = u32x2{w0, w1};
}
__device__ __forceinline__ uint32_t load_mask8(const uint8_t* p) {
  const u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
  uint32_t bits = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    bits |= (((w.x >> (8 * j)) & 0xffu) ? 1u : 0u) << j;
    bits |= (((w.y >> (8 * j)) & 0xffu) ? 1u : 0u) << (4 + j);
  }
  return bits;
}

// 8 consecutive elements of T <-> 8 floats
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* f) {
  VecIO<T>::unpack(ld16(p), f);
  if constexpr (VecIO<T>::N == 4) VecIO<T>::unpack(ld16(p + 4), f + 4);
}
template <typename T>
__device__ __forceinline__ void load8_keep(const T* p, float* f) {
  VecIO<T>::unpack(ld16_keep(p), f);
  if constexpr (VecIO<T>::N == 4) VecIO<T>::unpack(ld16_keep(p + 4), f + 4);
}
// STREAM is a template argument on purpose: with the choice as a run-time flag the compiler merges the two
// branches into one plain store and the non-temporal hint is lost.
template <typename T, bool STREAM>
__device__ __forceinline__ void store8(T* p, const float* f) {
  if constexpr (STREAM) {
    st16_stream(p, VecIO<T>::pack(f));
    if constexpr (VecIO<T>::N == 4) st16_stream(p + 4, VecIO<T>::pack(f + 4));
  } else {
    st16(p, VecIO<T>::pack(f));
    if constexpr (VecIO<T>::N == 4) st16(p + 4, VecIO<T>::pack(f + 4));
  }
}

constexpr int kChunk = 8;

// 1-based row number of a subset entry, 0 when it names no row or lies outside [0, numrows]
__device__ __forceinline__ int64_t subset_row(const int32_t* subset, int64_t row, int64_t numrows) {
  const int64_t v = subset[row];
  return (v < 0 || v > numrows) ? 0 : v;
}

// ===========================================================================
// forward
// ===========================================================================
struct DalFwdArgs {
  const void* x0;
  const void* x1;
  const void* residual;
  const void* gamma;
  const void* beta;
  const void* gamma1;
  const void* beta1;
  const void* rowscale;
  const void* colscale;
  const int32_t* x0_subset;
  const int32_t* z_subset;
  void* z;
  void* z1;
  void* x;
  uint8_t* dmask;
  uint8_t* dmask1;
  float* mu;
  float* rs;
  int64_t rows, x0_numrows, z_numrows;
  int cols, nchunks, tpr;
  float eps, inv_cols, scale, rowscale_const;
  int is_rms, dropout;
  DropArgs drop;
};

// IT / RT / WT: input, residual and weight element types; NC: chunks per thread.  A block holds
// blockDim.x / tpr row groups; every group takes part in the (block-wide) reduction barrier, a group
// past the last row works on a copy of the last row and stores nothing.
template <typename IT, typename RT, typename WT, int NC>
__global__ __launch_bounds__(256)
void dal_fwd_kernel(DalFwdArgs a) {
  __shared__ float red[kMaxWaves * 3];
  const int tpr = a.tpr;
  const int group = __builtin_amdgcn_readfirstlane(int(threadIdx.x) / tpr);
  const int t = int(threadIdx.x) - group * tpr;
  const int rpb = int(blockDim.x) / tpr;
  const int wpg = tpr >> 6;
  const int64_t row_raw = int64_t(blockIdx.x) * rpb + group;
  const bool row_ok = row_raw < a.rows;
  const int64_t row = row_ok ? row_raw : a.rows - 1;

  const bool subset = a.x0_subset != nullptr;
  float rowscale_val = 1.f;
  int64_t row_x0 = row + 1, row_z = row + 1;
  if (subset) {
    rowscale_val = a.rowscale_const;
    row_x0 = subset_row(a.x0_subset, row, a.x0_numrows);
    row_z = subset_row(a.z_subset, row, a.z_numrows);
  } else if (a.rowscale) {
    rowscale_val = Cvt<IT>::load(static_cast<const IT*>(a.rowscale) + row);
  }
  const bool load_x0 = row_x0 > 0;
  const bool dropout = a.dropout != 0;

  // Every load of the row is issued before the first one is waited for (the optional operands sit behind
  // uniform branches; unpacking inside those branches would serialise the loads).  A thread past the row's
  // end shadows chunk 0 and contributes nothing.
  constexpr int NI = kChunk / VecIO<IT>::N;
  constexpr int NR = kChunk / VecIO<RT>::N;
  u32x4 raw0[NC][NI], raw1[NC][NI], rawr[NC][NR];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
#pragma unroll
    for (int k = 0; k < NI; ++k) { raw0[i][k] = u32x4{0, 0, 0, 0}; raw1[i][k] = u32x4{0, 0, 0, 0}; }
#pragma unroll
    for (int k = 0; k < NR; ++k) rawr[i][k] = u32x4{0, 0, 0, 0};
  }
  if (load_x0) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int c = i * tpr + t;
      const IT* p = static_cast<const IT*>(a.x0) + (row_x0 - 1) * int64_t(a.cols) + (c < a.nchunks ? c : 0) * kChunk;
#pragma unroll
      for (int k = 0; k < NI; ++k) raw0[i][k] = ld16(p + k * VecIO<IT>::N);
    }
  }
  if (a.x1) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int c = i * tpr + t;
      const IT* p = static_cast<const IT*>(a.x1) + row * int64_t(a.cols) + (c < a.nchunks ? c : 0) * kChunk;
#pragma unroll
      for (int k = 0; k < NI; ++k) raw1[i][k] = ld16(p + k * VecIO<IT>::N);
    }
  }
  if (a.residual) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int c = i * tpr + t;
      const RT* p = static_cast<const RT*>(a.residual) + row * int64_t(a.cols) + (c < a.nchunks ? c : 0) * kChunk;
#pragma unroll
      for (int k = 0; k < NR; ++k) rawr[i][k] = ld16(p + k * VecIO<RT>::N);
    }
  }

  float xf[NC * kChunk];
  int cnt = 0;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = i * tpr + t;
    float* v = &xf[i * kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; ++j) v[j] = 0.f;
    if (c < a.nchunks) {
      cnt += kChunk;
      const int col = c * kChunk;
      if (load_x0) {
        const int64_t e0 = (row_x0 - 1) * int64_t(a.cols) + col;
        uint32_t keep = 0xffu;
        if (dropout) {
          keep = keep_bits8(e0, 0, a.drop);
          if (row_ok) store_mask8(a.dmask + e0, keep);
        }
#pragma unroll
        for (int k = 0; k < NI; ++k) VecIO<IT>::unpack(raw0[i][k], v + k * VecIO<IT>::N);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
          float xv = v[j] * rowscale_val;
          if (dropout) xv = ((keep >> j) & 1u) ? xv * a.scale : 0.f;
          v[j] = xv;
        }
        if (a.colscale) {
          float cs[kChunk];
          load8_keep<WT>(static_cast<const WT*>(a.colscale) + col, cs);
#pragma unroll
          for (int j = 0; j < kChunk; ++j) v[j] *= cs[j];
        }
      }
      const int64_t e = row * int64_t(a.cols) + col;
      if (a.x1) {
        float w[kChunk];
        uint32_t keep = 0xffu;
        if (dropout) {
          keep = keep_bits8(e, 1, a.drop);
          if (row_ok) store_mask8(a.dmask1 + e, keep);
        }
#pragma unroll
        for (int k = 0; k < NI; ++k) VecIO<IT>::unpack(raw1[i][k], w + k * VecIO<IT>::N);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
          float xv = w[j];
          if (dropout) xv = ((keep >> j) & 1u) ? xv * a.scale : 0.f;
          v[j] += xv;
        }
      }
      if (a.residual) {
        float w[kChunk];
#pragma unroll
        for (int k = 0; k < NR; ++k) VecIO<RT>::unpack(rawr[i][k], w + k * VecIO<RT>::N);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) v[j] += w[j];
      }
      if (a.x && row_ok) store8<RT, false>(static_cast<RT*>(a.x) + e, v);
    }
  }

  const int first_wave = group * wpg;
  float mu, rs;
  if (a.is_rms) {
    SumTuple<2> s;
    s.v[0] = 0.f; s.v[1] = 0.f;
#pragma unroll
    for (int e = 0; e < NC * kChunk; ++e) { s.v[0] += xf[e]; s.v[1] = fmaf(xf[e], xf[e], s.v[1]); }
    s = group_allreduce_tuple(s, red, first_wave, wpg);
    mu = s.v[0] * a.inv_cols;
    rs = 1.0f / sqrtf(s.v[1] * a.inv_cols + a.eps);   // mean(x^2) = var + mu^2
  } else {
    // per-thread (count, mean, M2) of the chunks held; slots past the row's end were left out of cnt
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < NC * kChunk; ++e) s += xf[e];
    const float mean_t = cnt > 0 ? s / float(cnt) : 0.f;
    float m2 = 0.f;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      if (i * tpr + t < a.nchunks) {
#pragma unroll
        for (int j = 0; j < kChunk; ++j) { const float d = xf[i * kChunk + j] - mean_t; m2 = fmaf(d, d, m2); }
      }
    }
    MomentTuple m;
    m.v[0] = float(cnt); m.v[1] = mean_t; m.v[2] = m2;
    m = group_allreduce_tuple(m, red, first_wave, wpg);
    mu = m.v[1];
    rs = 1.0f / sqrtf(m.v[2] * a.inv_cols + a.eps);
  }
  if (t == 0 && row_ok) {
    a.mu[row] = mu;
    a.rs[row] = rs;
  }

  if (!row_ok || row_z <= 0) return;   // after the only barrier
  const float shift = a.is_rms ? 0.f : mu;
  const int64_t zbase = (row_z - 1) * int64_t(a.cols);
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = i * tpr + t;
    if (c < a.nchunks) {
      const int col = c * kChunk;
      float y[kChunk], g[kChunk], b[kChunk], o[kChunk];
#pragma unroll
      for (int j = 0; j < kChunk; ++j) { y[j] = rs * (xf[i * kChunk + j] - shift); b[j] = 0.f; }
      load8_keep<WT>(static_cast<const WT*>(a.gamma) + col, g);
      if (a.beta) load8_keep<WT>(static_cast<const WT*>(a.beta) + col, b);
#pragma unroll
      for (int j = 0; j < kChunk; ++j) o[j] = fmaf(g[j], y[j], b[j]);
      store8<IT, true>(static_cast<IT*>(a.z) + zbase + col, o);
      if (a.gamma1) {
#pragma unroll
        for (int j = 0; j < kChunk; ++j) b[j] = 0.f;
        load8_keep<WT>(static_cast<const WT*>(a.gamma1) + col, g);
        if (a.beta1) load8_keep<WT>(static_cast<const WT*>(a.beta1) + col, b);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) o[j] = fmaf(g[j], y[j], b[j]);
        store8<IT, true>(static_cast<IT*>(a.z1) + zbase + col, o);
      }
    }
  }
}

// ===========================================================================
// backward
// ===========================================================================
constexpr int kMaxParts = 5;   // dgamma, dbeta, dgamma1, dbeta1, dcolscale

struct DalBwdArgs {
  const void* dz;
  const void* dz1;
  const void* dx;
  const void* x;
  const void* x0;
  const uint8_t* dmask;
  const uint8_t* dmask1;
  const float* mu;
  const float* rs;
  const void* gamma;
  const void* gamma1;
  const void* rowscale;
  const void* colscale;
  const int32_t* x0_subset;
  const int32_t* z_subset;
  void* dx0;
  void* dx1;
  void* dresidual;
  float* part[kMaxParts];   // [groups of the grid, cols] each; nullptr: not wanted
  int64_t rows, x0_numrows, z_numrows;
  int cols, nchunks, tpr;
  float inv_cols, scale, rowscale_const;
  int is_rms, dropout;
};

// One chunk of 8 columns per thread.  COLSCALE: per-column scaling (and its gradient); G1: a second
// affine output (dz1 / gamma1 and their gradients).
template <typename IT, typename RT, typename WT, bool COLSCALE, bool G1>
__global__ __launch_bounds__(1024)
void dal_bwd_kernel(DalBwdArgs a) {
  __shared__ float red[2][kMaxWaves * 2];   // double-buffered by step parity
  const int tpr = a.tpr;
  const int group = __builtin_amdgcn_readfirstlane(int(threadIdx.x) / tpr);
  const int t = int(threadIdx.x) - group * tpr;
  const int rpb = int(blockDim.x) / tpr;
  const int wpg = tpr >> 6;
  const int first_wave = group * wpg;
  const bool in = t < a.nchunks;
  const int col = (in ? t : a.nchunks - 1) * kChunk;   // an idle thread shadows the last chunk, stores nothing
  const bool subset = a.x0_subset != nullptr;
  const bool dropout = a.dropout != 0;

  float g0[kChunk];
  [[maybe_unused]] float g1[G1 ? kChunk : 1];
  [[maybe_unused]] float cs[COLSCALE ? kChunk : 1];
  load8_keep<WT>(static_cast<const WT*>(a.gamma) + col, g0);
  if constexpr (G1) load8_keep<WT>(static_cast<const WT*>(a.gamma1) + col, g1);
  if constexpr (COLSCALE) load8_keep<WT>(static_cast<const WT*>(a.colscale) + col, cs);

  float dg0[kChunk], db0[kChunk];
  [[maybe_unused]] float dg1[G1 ? kChunk : 1], db1[G1 ? kChunk : 1], dcs[COLSCALE ? kChunk : 1];
#pragma unroll
  for (int j = 0; j < kChunk; ++j) {
    dg0[j] = 0.f; db0[j] = 0.f;
    if constexpr (G1) { dg1[j] = 0.f; db1[j] = 0.f; }
    if constexpr (COLSCALE) dcs[j] = 0.f;
  }

  const int64_t stride = int64_t(gridDim.x) * rpb;
  int parity = 0;
  // both loop bounds are block-uniform: every thread of the block reaches the barrier of every step
  for (int64_t base = int64_t(blockIdx.x) * rpb; base < a.rows; base += stride) {
    const int64_t row_raw = base + group;
    const bool row_ok = row_raw < a.rows;
    const int64_t row = row_ok ? row_raw : a.rows - 1;
    const float mu = a.is_rms ? 0.f : a.mu[row];
    const float rs = a.rs[row];
    float rowscale_val = 1.f;
    int64_t row_x0 = row + 1, row_z = row + 1;
    if (subset) {
      rowscale_val = a.rowscale_const;
      row_x0 = subset_row(a.x0_subset, row, a.x0_numrows);
      row_z = subset_row(a.z_subset, row, a.z_numrows);
    } else if (a.rowscale) {
      rowscale_val = Cvt<IT>::load(static_cast<const IT*>(a.rowscale) + row);
    }
    const bool load_dz = row_z > 0;
    const bool save_dx0 = row_x0 > 0;
    const bool live = row_ok && in;
    const int64_t e = row * int64_t(a.cols) + col;

    float dz[kChunk], y[kChunk], dy[kChunk];
    [[maybe_unused]] float dz1[G1 ? kChunk : 1];
#pragma unroll
    for (int j = 0; j < kChunk; ++j) { dz[j] = 0.f; y[j] = 0.f; }
    if (load_dz) {
      load8<IT>(static_cast<const IT*>(a.dz) + (row_z - 1) * int64_t(a.cols) + col, dz);
      float xv[kChunk];
      load8<RT>(static_cast<const RT*>(a.x) + e, xv);
#pragma unroll
      for (int j = 0; j < kChunk; ++j) y[j] = rs * (xv[j] - mu);
    }
    if constexpr (G1) load8<IT>(static_cast<const IT*>(a.dz1) + e, dz1);
    SumTuple<2> s;
    s.v[0] = 0.f; s.v[1] = 0.f;
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      const float d0 = live ? dz[j] : 0.f;
      float d = g0[j] * d0;
      dg0[j] = fmaf(d0, y[j], dg0[j]);
      db0[j] += d0;
      if constexpr (G1) {
        const float d1 = live ? dz1[j] : 0.f;
        d = fmaf(g1[j], d1, d);
        dg1[j] = fmaf(d1, y[j], dg1[j]);
        db1[j] += d1;
      }
      dy[j] = d;
      s.v[0] += d;
      s.v[1] = fmaf(d, y[j], s.v[1]);
    }
    s = group_allreduce_tuple(s, red[parity], first_wave, wpg);
    parity ^= 1;
    if (!live) continue;   // no barrier below this point

    const float mdy = a.is_rms ? 0.f : s.v[0] * a.inv_cols;
    const float mdyy = s.v[1] * a.inv_cols;
    float dxr[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; ++j) dxr[j] = rs * (dy[j] - fmaf(mdyy, y[j], mdy));
    if (a.dx) {
      float u[kChunk];
      load8<RT>(static_cast<const RT*>(a.dx) + e, u);
#pragma unroll
      for (int j = 0; j < kChunk; ++j) dxr[j] += u[j];
    }
    if (a.dresidual) store8<RT, false>(static_cast<RT*>(a.dresidual) + e, dxr);
    if (save_dx0) {
      const int64_t e0 = (row_x0 - 1) * int64_t(a.cols) + col;
      uint32_t keep = 0xffu;
      float o[kChunk];
#pragma unroll
      for (int j = 0; j < kChunk; ++j) o[j] = dxr[j] * rowscale_val;
      if (dropout) {
        keep = load_mask8(a.dmask + e0);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) o[j] *= a.scale;
      }
      if constexpr (COLSCALE) {
        float xv0[kChunk];
        load8<IT>(static_cast<const IT*>(a.x0) + e0, xv0);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
          const bool k = (keep >> j) & 1u;
          dcs[j] += k ? o[j] * xv0[j] : 0.f;
          o[j] *= cs[j];
        }
      }
#pragma unroll
      for (int j = 0; j < kChunk; ++j) o[j] = ((keep >> j) & 1u) ? o[j] : 0.f;
      store8<IT, true>(static_cast<IT*>(a.dx0) + e0, o);
    }
    if (a.dx1) {
      float o[kChunk];
      uint32_t keep = 0xffu;
      if (dropout) keep = load_mask8(a.dmask1 + e);
#pragma unroll
      for (int j = 0; j < kChunk; ++j) {
        const float v = dropout ? dxr[j] * a.scale : dxr[j];
        o[j] = ((keep >> j) & 1u) ? v : 0.f;
      }
      store8<IT, true>(static_cast<IT*>(a.dx1) + e, o);
    }
  }

  if (!in) return;
  const int64_t prow = (int64_t(blockIdx.x) * rpb + group) * a.cols + col;
  auto put = [&](float* part, const float* acc) {
    if (part == nullptr) return;
    st16(part + prow, VecIO<float>::pack(acc));
    st16(part + prow + 4, VecIO<float>::pack(acc + 4));
  };
  put(a.part[0], dg0);
  put(a.part[1], db0);
  if constexpr (G1) { put(a.part[2], dg1); put(a.part[3], db1); }
  if constexpr (COLSCALE) put(a.part[4], dcs);
}

// The pre-norm residual block's backward, the shape a transformer layer calls: dropout on, the gradient of
// the residual stream coming in (dx) and going out (dresidual), no scaling, no subsets, one affine pair, and
// a row that fills every thread's chunk exactly.  With nothing optional left, the row loop holds no branch
// around a memory instruction, so the compiler counts outstanding loads exactly and PF rows stay in flight
// per thread group (a ring of register slots refilled as soon as a slot has been unpacked); rows past the
// end are clamped to the last row and their results dropped.
// TPR: the group width when the one group of a block is the whole block and its size is known at compile time
// (512 threads = 4096 columns), else 0: the launch bound and the cross-wavefront step of the row sums follow it.
template <typename IT, typename RT, typename WT, int PF, int TPR>
__global__ __launch_bounds__(TPR ? TPR : 1024)
void dal_bwd_stream_kernel(DalBwdArgs a) {
  constexpr int NI = kChunk / VecIO<IT>::N;   // 16-byte vectors per chunk of the input type
  constexpr int NR = kChunk / VecIO<RT>::N;   //                       ... of the residual type
  __shared__ __align__(16) float red[2][kMaxWaves * 2];
  const int tpr = TPR ? TPR : a.tpr;
  const int group = TPR ? 0 : __builtin_amdgcn_readfirstlane(int(threadIdx.x) / tpr);
  const int t = int(threadIdx.x) - group * tpr;
  const int rpb = TPR ? 1 : int(blockDim.x) / tpr;
  const int wpg = tpr >> 6;
  const int first_wave = group * wpg;
  const int col = t * kChunk;

  float g0[kChunk];
  load8_keep<WT>(static_cast<const WT*>(a.gamma) + col, g0);
  float dg0[kChunk], db0[kChunk];
#pragma unroll
  for (int j = 0; j < kChunk; ++j) { dg0[j] = 0.f; db0[j] = 0.f; }

  const int64_t stride = int64_t(gridDim.x) * rpb;
  const int64_t last_row = a.rows - 1;
  u32x4 ndz[PF][NI], nx[PF][NR], ndx[PF][NR];
  u32x2 nm[PF];
  float nmu[PF], nrs[PF];
  auto issue = [&](auto slot, int64_t r) {
    constexpr int d = decltype(slot)::value;
    const int64_t rc = r < last_row ? r : last_row;
    const int64_t e = rc * int64_t(a.cols) + col;
    nmu[d] = a.mu[rc];
    nrs[d] = a.rs[rc];
#pragma unroll
    for (int i = 0; i < NI; ++i) ndz[d][i] = ld16(static_cast<const IT*>(a.dz) + e + i * VecIO<IT>::N);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      nx[d][i] = ld16(static_cast<const RT*>(a.x) + e + i * VecIO<RT>::N);
      ndx[d][i] = ld16(static_cast<const RT*>(a.dx) + e + i * VecIO<RT>::N);
    }
    nm[d] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(a.dmask + e));
  };
  int64_t row0 = int64_t(blockIdx.x) * rpb + group;
  static_for<PF>([&](auto slot) { issue(slot, row0 + decltype(slot)::value * stride); });

  int parity = 0;
  auto step = [&](auto slot, auto guarded) {
    constexpr int d = decltype(slot)::value;
    constexpr bool GUARD = decltype(guarded)::value;
    const int64_t row = row0 + d * stride;
    const bool valid = !GUARD || row < a.rows;
    float dz[kChunk], y[kChunk], u[kChunk];
#pragma unroll
    for (int i = 0; i < NI; ++i) VecIO<IT>::unpack(ndz[d][i], &dz[i * VecIO<IT>::N]);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      VecIO<RT>::unpack(nx[d][i], &y[i * VecIO<RT>::N]);
      VecIO<RT>::unpack(ndx[d][i], &u[i * VecIO<RT>::N]);
    }
    const u32x2 mw = nm[d];
    const float mu = a.is_rms ? 0.f : nmu[d];
    const float rs = nrs[d];
    issue(slot, row + int64_t(PF) * stride);   // the slot is free again

    SumTuple<2> s;
    s.v[0] = 0.f; s.v[1] = 0.f;
    float dy[kChunk];
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      const float d0 = (GUARD && !valid) ? 0.f : dz[j];
      y[j] = rs * (y[j] - mu);
      dy[j] = g0[j] * d0;
      dg0[j] = fmaf(d0, y[j], dg0[j]);
      db0[j] += d0;
      s.v[0] += dy[j];
      s.v[1] = fmaf(dy[j], y[j], s.v[1]);
    }
    if constexpr (TPR != 0) s = group_allreduce_tuple_fixed<SumTuple<2>, TPR / 64>(s, red[parity]);
    else s = group_allreduce_tuple(s, red[parity], first_wave, wpg);
    parity ^= 1;
    if (valid) {
      const float mdy = a.is_rms ? 0.f : s.v[0] * a.inv_cols;
      const float mdyy = s.v[1] * a.inv_cols;
      float o[kChunk];
#pragma unroll
      for (int j = 0; j < kChunk; ++j) {
        u[j] += rs * (dy[j] - fmaf(mdyy, y[j], mdy));
        const uint32_t byte = ((j < 4 ? mw.x : mw.y) >> (8 * (j & 3))) & 0xffu;
        o[j] = byte ? u[j] * a.scale : 0.f;
      }
      const int64_t e = row * int64_t(a.cols) + col;
      store8<RT, false>(static_cast<RT*>(a.dresidual) + e, u);
      store8<IT, true>(static_cast<IT*>(a.dx0) + e, o);
    }
  };
  int64_t base = int64_t(blockIdx.x) * rpb;
  const int64_t round = int64_t(PF) * stride;
  // rounds in which every slot of every group of this block holds an existing row, then the guarded tail;
  // both bounds are block-uniform, so every thread reaches the barrier of every step
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

  const int64_t prow = (int64_t(blockIdx.x) * rpb + group) * a.cols + col;
  if (a.part[0]) {
    st16(a.part[0] + prow, VecIO<float>::pack(dg0));
    st16(a.part[0] + prow + 4, VecIO<float>::pack(dg0 + 4));
  }
  if (a.part[1]) {
    st16(a.part[1] + prow, VecIO<float>::pack(db0));
    st16(a.part[1] + prow + 4, VecIO<float>::pack(db0 + 4));
  }
}

// Folds [nparts, cols] fp32 partial rows into a [cols] vector of WT; blockIdx.y picks which of the
// (up to five) sums.  A block covers 128 columns as 32 float4 column groups x 16 row slices.
struct DalFoldArgs {
  const float* part[kMaxParts];
  void* out[kMaxParts];
  int nparts, cols;
};

template <typename WT>
__global__ __launch_bounds__(512)
void dal_fold_kernel(DalFoldArgs a) {
  __shared__ float lds[16][32][4];
  const float* part = a.part[blockIdx.y];
  WT* out = static_cast<WT*>(a.out[blockIdx.y]);
  if (part == nullptr || out == nullptr) return;   // uniform over the block
  const int cg = threadIdx.x & 31, slice = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + cg) * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < a.cols) {
    for (int r = slice; r < a.nparts; r += 16) {
      const u32x4 v = ld16_keep(part + int64_t(r) * a.cols + c);
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
    if (oc < a.cols) Cvt<WT>::store(out + oc, s);
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
template <typename T> struct TypeTag { using type = T; };

// the (weight, input, residual) combinations the reference registers kernels for
template <typename F>
static int dispatch_types(int wtype, int itype, int rtype, const char* who, F&& f) {
#define HK_DAL_CASE(W, I, R, WT, IT, RT) \
  if (wtype == W && itype == I && rtype == R) return f(TypeTag<IT>{}, TypeTag<RT>{}, TypeTag<WT>{})
  HK_DAL_CASE(HK_FLOAT32, HK_FLOAT32, HK_FLOAT32, float, float, float);
  HK_DAL_CASE(HK_FLOAT16, HK_FLOAT16, HK_FLOAT16, fp16, fp16, fp16);
  HK_DAL_CASE(HK_BFLOAT16, HK_BFLOAT16, HK_BFLOAT16, bf16, bf16, bf16);
  HK_DAL_CASE(HK_FLOAT32, HK_FLOAT16, HK_FLOAT32, float, fp16, float);
  HK_DAL_CASE(HK_FLOAT32, HK_BFLOAT16, HK_FLOAT32, float, bf16, float);
  HK_DAL_CASE(HK_FLOAT16, HK_FLOAT16, HK_FLOAT32, fp16, fp16, float);
  HK_DAL_CASE(HK_BFLOAT16, HK_BFLOAT16, HK_FLOAT32, bf16, bf16, float);
  HK_DAL_CASE(HK_FLOAT32, HK_FLOAT16, HK_FLOAT16, float, fp16, fp16);
  HK_DAL_CASE(HK_FLOAT32, HK_BFLOAT16, HK_BFLOAT16, float, bf16, bf16);
  HK_DAL_CASE(HK_FLOAT16, HK_FLOAT32, HK_FLOAT32, fp16, float, float);
#undef HK_DAL_CASE
  set_last_error("%s: no kernel for weight dtype %d, input dtype %d, residual dtype %d", who, wtype, itype,
                 rtype);
  return HK_ERR_UNSUPPORTED;
}

static bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

struct BwdShape {
  int tpr, rpb, block, grid;
  int64_t nparts;
};

static BwdShape plan_dal_bwd(int64_t rows, int cols) {
  BwdShape p{};
  const int nchunks = cols / kChunk;
  p.tpr = (nchunks + 63) / 64 * 64;
  p.rpb = p.tpr > 512 ? 1 : 512 / p.tpr;
  const int forced_rpb = tune_get(TUNE_NORM_BWD_ROWS_PER_BLOCK);
  if (forced_rpb > 0) p.rpb = std::max(1, std::min(forced_rpb, 1024 / p.tpr));
  p.block = p.tpr * p.rpb;
  // two 512-thread workgroups (one of 1024) per compute unit
  int64_t grid = int64_t(device_cu_count()) * (p.block > 512 ? 1 : 2);
  if (tune_get(TUNE_NORM_BWD_BLOCKS) > 0) grid = tune_get(TUNE_NORM_BWD_BLOCKS);
  const int64_t useful = (rows + p.rpb - 1) / p.rpb;
  if (grid > useful) grid = useful;
  if (grid < 1) grid = 1;
  p.grid = int(grid);
  p.nparts = grid * p.rpb;
  return p;
}

static int count_parts(const hkDropoutAddLnBwdParams& p) {
  // slots are fixed (dgamma, dbeta, dgamma1, dbeta1, dcolscale); the workspace holds the highest one in use
  int n = 0;
  if (p.dgamma) n = 1;
  if (p.dbeta) n = 2;
  if (p.dgamma1) n = 3;
  if (p.dbeta1) n = 4;
  if (p.dcolscale) n = 5;
  return n;
}

static int check_common(const char* who, int64_t rows, int64_t cols, float dropout_p) {
  HK_REQUIRE(rows >= 0 && cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  HK_REQUIRE(rows <= 0x7fffffffLL, HK_ERR_INVALID, "%s: too many rows (%lld)", who, (long long) rows);
  HK_REQUIRE(cols % 8 == 0 && cols <= 8192, HK_ERR_INVALID,
             "%s: hidden size must be a multiple of 8 and at most 8192, got %lld", who, (long long) cols);
  HK_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, HK_ERR_INVALID, "%s: dropout_p %g outside [0, 1)", who,
             double(dropout_p));
  return HK_OK;
}

} // namespace hk

using namespace hk;

extern "C" {

int hk_dropout_add_ln_fwd_ex(const hkDropoutAddLnFwdParams* pp, hkStream_t stream) {
  const char* who = "hk_dropout_add_ln_fwd_ex";
  HK_REQUIRE(pp != nullptr, HK_ERR_INVALID, "%s: null parameter block", who);
  const hkDropoutAddLnFwdParams& p = *pp;
  int rc = check_common(who, p.rows, p.cols, p.dropout_p);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(p.epsilon >= 0.f, HK_ERR_INVALID, "%s: epsilon must be >= 0", who);
  const bool subset = p.x0_subset != nullptr || p.z_subset != nullptr;
  const bool parallel = p.x1 != nullptr || p.gamma1 != nullptr || p.z1 != nullptr || p.beta1 != nullptr ||
                        p.dmask1 != nullptr;
  HK_REQUIRE(!subset || (p.x0_subset && p.z_subset), HK_ERR_INVALID,
             "%s: x0_subset and z_subset come together", who);
  HK_REQUIRE(!subset || (p.x0_numrows >= 0 && p.z_numrows >= 0), HK_ERR_INVALID,
             "%s: negative x0_numrows / z_numrows", who);
  HK_REQUIRE(!(parallel && (subset || p.rowscale || p.colscale)), HK_ERR_UNSUPPORTED,
             "%s: the parallel-residual form takes no rowscale, colscale or row subsets", who);
  HK_REQUIRE(!p.gamma1 || p.z1, HK_ERR_INVALID, "%s: gamma1 given without z1", who);
  HK_REQUIRE(!(p.z1 || p.beta1) || p.gamma1, HK_ERR_INVALID, "%s: z1 / beta1 given without gamma1", who);
  if (p.rows == 0 || p.cols == 0) return HK_OK;
  HK_REQUIRE(p.x0 && p.gamma && p.z && p.mu && p.rs, HK_ERR_INVALID, "%s: null input/output", who);
  const bool dropout = p.dropout_p > 0.f;
  HK_REQUIRE(!dropout || p.dmask, HK_ERR_INVALID, "%s: dmask is required when dropout_p > 0", who);
  HK_REQUIRE(!dropout || !p.x1 || p.dmask1, HK_ERR_INVALID,
             "%s: dmask1 is required when dropout_p > 0 and x1 is given", who);
  HK_REQUIRE(aligned16(p.x0) && aligned16(p.x1) && aligned16(p.residual) && aligned16(p.gamma) &&
                 aligned16(p.beta) && aligned16(p.gamma1) && aligned16(p.beta1) && aligned16(p.colscale) &&
                 aligned16(p.z) && aligned16(p.z1) && aligned16(p.x) && aligned8(p.dmask) && aligned8(p.dmask1),
             HK_ERR_INVALID, "%s: data pointers must be 16-byte aligned (masks 8-byte)", who);

  // nothing beyond the plain interface: the tuned row kernels take it
  const bool plain = !dropout && !subset && !parallel && !p.rowscale && !p.colscale &&
                     p.itype == p.rtype && p.itype == p.wtype;
  if (plain) {
    return hk_dropout_add_ln_fwd(p.itype, p.rtype, p.wtype, p.x0, p.residual, p.gamma, p.beta, p.z, p.x, p.mu,
                                 p.rs, p.rows, p.cols, p.epsilon, p.is_rms_norm, stream);
  }

  DalFwdArgs a{};
  a.x0 = p.x0; a.x1 = p.x1; a.residual = p.residual; a.gamma = p.gamma; a.beta = p.beta;
  a.gamma1 = p.gamma1; a.beta1 = p.beta1; a.rowscale = subset ? nullptr : p.rowscale; a.colscale = p.colscale;
  a.x0_subset = p.x0_subset; a.z_subset = p.z_subset;
  a.z = p.z; a.z1 = p.z1; a.x = p.x; a.dmask = p.dmask; a.dmask1 = p.dmask1; a.mu = p.mu; a.rs = p.rs;
  a.rows = p.rows; a.x0_numrows = subset ? p.x0_numrows : p.rows; a.z_numrows = subset ? p.z_numrows : p.rows;
  a.cols = int(p.cols); a.nchunks = int(p.cols) / kChunk;
  a.eps = p.epsilon; a.inv_cols = 1.0f / float(p.cols);
  a.scale = 1.0f / (1.0f - p.dropout_p); a.rowscale_const = p.rowscale_const;
  a.is_rms = p.is_rms_norm ? 1 : 0; a.dropout = dropout ? 1 : 0;
  a.drop.seed_lo = uint32_t(p.seed); a.drop.seed_hi = uint32_t(p.seed >> 32);
  a.drop.off_lo = uint32_t(p.offset); a.drop.off_hi = uint32_t(p.offset >> 32);
  a.drop.keep_p = 1.0f - p.dropout_p;

  // chunks per thread: the fewest that keep a row within 256 threads
  const int nc = a.nchunks <= 256 ? 1 : (a.nchunks <= 512 ? 2 : 4);
  a.tpr = ((a.nchunks + nc - 1) / nc + 63) / 64 * 64;
  const int rpb = std::max(1, 256 / a.tpr);
  const dim3 block{unsigned(a.tpr * rpb)}, grid{unsigned((p.rows + rpb - 1) / rpb)};
  hipStream_t s = as_hip(stream);
  return dispatch_types(p.wtype, p.itype, p.rtype, who, [&](auto it, auto rt, auto wt) {
    using IT = typename decltype(it)::type;
    using RT = typename decltype(rt)::type;
    using WT = typename decltype(wt)::type;
    profile_before(s);
    switch (nc) {
      case 1: HK_LAUNCH((dal_fwd_kernel<IT, RT, WT, 1>), grid, block, 0, s, a); break;
      case 2: HK_LAUNCH((dal_fwd_kernel<IT, RT, WT, 2>), grid, block, 0, s, a); break;
      default: HK_LAUNCH((dal_fwd_kernel<IT, RT, WT, 4>), grid, block, 0, s, a); break;
    }
    profile_after(s);
    return launch_check("dal_fwd_kernel");
  });
}

int hk_dropout_add_ln_bwd_ex_workspace_bytes(const hkDropoutAddLnBwdParams* pp, size_t* bytes) {
  const char* who = "hk_dropout_add_ln_bwd_ex_workspace_bytes";
  HK_REQUIRE(pp != nullptr && bytes != nullptr, HK_ERR_INVALID, "%s: null argument", who);
  const hkDropoutAddLnBwdParams& p = *pp;
  *bytes = 0;
  int rc = check_common(who, p.rows, p.cols, p.dropout_p);
  if (rc != HK_OK) return rc;
  if (p.rows == 0 || p.cols == 0) return HK_OK;
  const BwdShape sh = plan_dal_bwd(p.rows, int(p.cols));
  size_t general = size_t(count_parts(p)) * size_t(sh.nparts) * size_t(p.cols) * sizeof(float);
  // a call without extra features is handed to the plain backward, which sizes its own scratch
  size_t plain = 0;
  if (p.itype == p.rtype && p.itype == p.wtype) {
    rc = hk_norm_bwd_workspace_bytes(p.itype, p.rows, p.cols, &plain);
    if (rc != HK_OK) return rc;
  }
  *bytes = std::max(general, plain);
  return HK_OK;
}

int hk_dropout_add_ln_bwd_ex(const hkDropoutAddLnBwdParams* pp, hkStream_t stream) {
  const char* who = "hk_dropout_add_ln_bwd_ex";
  HK_REQUIRE(pp != nullptr, HK_ERR_INVALID, "%s: null parameter block", who);
  const hkDropoutAddLnBwdParams& p = *pp;
  int rc = check_common(who, p.rows, p.cols, p.dropout_p);
  if (rc != HK_OK) return rc;
  const bool subset = p.x0_subset != nullptr || p.z_subset != nullptr;
  const bool g1 = p.gamma1 != nullptr;
  const bool parallel = g1 || p.dz1 != nullptr || p.dx1 != nullptr || p.dmask1 != nullptr ||
                        p.dgamma1 != nullptr || p.dbeta1 != nullptr;
  const bool colscale = p.colscale != nullptr;
  HK_REQUIRE(!subset || (p.x0_subset && p.z_subset), HK_ERR_INVALID,
             "%s: x0_subset and z_subset come together", who);
  HK_REQUIRE(!subset || (p.x0_numrows >= 0 && p.z_numrows >= 0), HK_ERR_INVALID,
             "%s: negative x0_numrows / z_numrows", who);
  HK_REQUIRE(!(parallel && (subset || p.rowscale || colscale)), HK_ERR_UNSUPPORTED,
             "%s: the parallel-residual form takes no rowscale, colscale or row subsets", who);
  HK_REQUIRE(!g1 || p.dz1, HK_ERR_INVALID, "%s: gamma1 given without dz1", who);
  HK_REQUIRE(!(p.dz1 || p.dgamma1 || p.dbeta1) || g1, HK_ERR_INVALID,
             "%s: dz1 / dgamma1 / dbeta1 given without gamma1", who);
  HK_REQUIRE(colscale || !p.dcolscale, HK_ERR_INVALID, "%s: dcolscale given without colscale", who);
  hipStream_t s = as_hip(stream);
  if (p.cols == 0) return HK_OK;
  if (p.rows == 0) {
    // no rows: the column sums are empty sums
    const size_t wbytes = size_t(p.cols) * ((p.wtype == HK_FLOAT32) ? 4 : 2);
    void* outs[kMaxParts] = {p.dgamma, p.dbeta, p.dgamma1, p.dbeta1, p.dcolscale};
    for (void* o : outs) {
      if (o) {
        rc = hk_memset(o, 0, wbytes, stream);
        if (rc != HK_OK) return rc;
      }
    }
    return HK_OK;
  }
  HK_REQUIRE(p.dz && p.x && p.mu && p.rs && p.gamma && p.dx0, HK_ERR_INVALID, "%s: null input/output", who);
  const bool dropout = p.dropout_p > 0.f;
  HK_REQUIRE(!dropout || p.dmask, HK_ERR_INVALID, "%s: dmask is required when dropout_p > 0", who);
  HK_REQUIRE(!dropout || !p.dx1 || p.dmask1, HK_ERR_INVALID,
             "%s: dmask1 is required when dropout_p > 0 and dx1 is wanted", who);
  HK_REQUIRE(!colscale || p.x0, HK_ERR_INVALID, "%s: x0 is required with colscale", who);
  HK_REQUIRE(aligned16(p.dz) && aligned16(p.dz1) && aligned16(p.dx) && aligned16(p.x) && aligned16(p.x0) &&
                 aligned16(p.gamma) && aligned16(p.gamma1) && aligned16(p.colscale) && aligned16(p.dx0) &&
                 aligned16(p.dx1) && aligned16(p.dresidual) && aligned8(p.dmask) && aligned8(p.dmask1),
             HK_ERR_INVALID, "%s: data pointers must be 16-byte aligned (masks 8-byte)", who);

  const bool plain = !dropout && !subset && !parallel && !p.rowscale && !colscale &&
                     p.itype == p.rtype && p.itype == p.wtype;
  if (plain) {
    return hk_dropout_add_ln_bwd(p.itype, p.rtype, p.wtype, p.dz, p.dx, p.x, p.mu, p.rs, p.gamma, p.dx0,
                                 p.dresidual, p.dgamma, p.dbeta, p.rows, p.cols, p.is_rms_norm, p.workspace,
                                 p.workspace_bytes, stream);
  }

  BwdShape sh = plan_dal_bwd(p.rows, int(p.cols));
  // the pre-norm residual block with full rows has a kernel of its own; it keeps two rows in flight per
  // thread group and runs best with one workgroup per compute unit (measured: 264 us against 283 us with
  // two at [32768 x 4096] bf16).  The workspace was sized for the larger grid.
  const bool stream_form = dropout && p.dx && p.dresidual && !subset && !p.rowscale && !colscale && !parallel &&
                           int(p.cols) / kChunk == sh.tpr && tune_get(TUNE_NORM_BWD_PREFETCH) != 1;
  if (stream_form && tune_get(TUNE_NORM_BWD_BLOCKS) <= 0 && sh.grid > device_cu_count()) {
    sh.grid = device_cu_count();
    sh.nparts = int64_t(sh.grid) * sh.rpb;
  }
  const int nslots = count_parts(p);
  const size_t slot_floats = size_t(sh.nparts) * size_t(p.cols);
  const size_t need = size_t(nslots) * slot_floats * sizeof(float);
  if (nslots > 0) {
    HK_REQUIRE(p.workspace != nullptr && p.workspace_bytes >= need, HK_ERR_WORKSPACE,
               "%s: workspace of %zu bytes needed, %zu given", who, need, p.workspace_bytes);
    HK_REQUIRE(aligned16(p.workspace), HK_ERR_INVALID, "%s: workspace must be 16-byte aligned", who);
  }

  DalBwdArgs a{};
  a.dz = p.dz; a.dz1 = p.dz1; a.dx = p.dx; a.x = p.x; a.x0 = p.x0; a.dmask = p.dmask; a.dmask1 = p.dmask1;
  a.mu = p.mu; a.rs = p.rs; a.gamma = p.gamma; a.gamma1 = p.gamma1;
  a.rowscale = subset ? nullptr : p.rowscale; a.colscale = p.colscale;
  a.x0_subset = p.x0_subset; a.z_subset = p.z_subset;
  a.dx0 = p.dx0; a.dx1 = p.dx1; a.dresidual = p.dresidual;
  void* outs[kMaxParts] = {p.dgamma, p.dbeta, p.dgamma1, p.dbeta1, p.dcolscale};
  for (int k = 0; k < kMaxParts; ++k)
    a.part[k] = outs[k] ? static_cast<float*>(p.workspace) + size_t(k) * slot_floats : nullptr;
  a.rows = p.rows; a.x0_numrows = subset ? p.x0_numrows : p.rows; a.z_numrows = subset ? p.z_numrows : p.rows;
  a.cols = int(p.cols); a.nchunks = int(p.cols) / kChunk; a.tpr = sh.tpr;
  a.inv_cols = 1.0f / float(p.cols); a.scale = 1.0f / (1.0f - p.dropout_p); a.rowscale_const = p.rowscale_const;
  a.is_rms = p.is_rms_norm ? 1 : 0; a.dropout = dropout ? 1 : 0;

  DalFoldArgs f{};
  for (int k = 0; k < kMaxParts; ++k) { f.part[k] = a.part[k]; f.out[k] = outs[k]; }
  f.nparts = int(sh.nparts); f.cols = int(p.cols);

  const dim3 grid{unsigned(sh.grid)}, block{unsigned(sh.block)};
  return dispatch_types(p.wtype, p.itype, p.rtype, who, [&](auto it, auto rt, auto wt) {
    using IT = typename decltype(it)::type;
    using RT = typename decltype(rt)::type;
    using WT = typename decltype(wt)::type;
    profile_before(s);
    // two rows in flight where the ring fits the registers (a 16-bit residual stream), else one
    constexpr int PF = sizeof(RT) == 2 ? 2 : 1;
    if (stream_form && sh.tpr == 512 && sh.block == 512) HK_LAUNCH((dal_bwd_stream_kernel<IT, RT, WT, PF, 512>), grid, block, 0, s, a);
    else if (stream_form) HK_LAUNCH((dal_bwd_stream_kernel<IT, RT, WT, PF, 0>), grid, block, 0, s, a);
    else if (g1) HK_LAUNCH((dal_bwd_kernel<IT, RT, WT, false, true>), grid, block, 0, s, a);
    else if (colscale) HK_LAUNCH((dal_bwd_kernel<IT, RT, WT, true, false>), grid, block, 0, s, a);
    else HK_LAUNCH((dal_bwd_kernel<IT, RT, WT, false, false>), grid, block, 0, s, a);
    profile_after(s);
    int r = launch_check("dal_bwd_kernel");
    if (r != HK_OK || nslots == 0) return r;
    HK_LAUNCH((dal_fold_kernel<WT>), dim3(unsigned((p.cols + 127) / 128), kMaxParts), dim3(512), 0, s, f);
    return launch_check("dal_fold_kernel");
  });
}

} // extern "C"
