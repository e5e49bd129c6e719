// LayerNorm / RMSNorm backward kernels and their launch logic, included by the per-type instantiation files.
//
// A persistent grid walks the rows; every thread owns a fixed set of columns, keeps the dgamma / dbeta column
// sums of its rows in registers, and the workgroup writes ONE fp32 partial row per block which a small second
// kernel folds into dgamma / dbeta.
#pragma once

#include "hk_norm.h"

namespace hk {

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
// past the row's end, STATS_F32 fixes the statistics' type, EXTRA says whether the
// optional operands (an upstream gradient added to dx, a second copy of dx) exist
// at all.  Only then does the compiler count outstanding loads exactly; any branch
// around a load in the loop makes it wait for all of them at every step, which
// flattens the ring to depth one.  Rows that do not fill a whole round of PF steps
// go through the same step with its guards switched on.
//
// MAXT is the launch bound: the register budget follows the block size the plan
// really uses (a 640-thread block of the 5120-column LayerNorm may hold 170
// registers per lane where a 1024-thread block may hold 128), which is what lets
// the LayerNorm modes, with the mean in their ring as well, keep two rows in flight.
//
// FIXED says that one group of exactly MAXT threads is the whole block: the group's
// width, and with it the number of wavefront partials every thread adds up after the
// barrier, is then a constant and the cross-wavefront step is straight-line code.
// Whatever the hot case never has is decided at compile time there: EXTRA also stands
// for "gamma clamped in dx on request" (a uniform branch between two copies of the
// arithmetic otherwise, whose merge costs one register move per live value per row);
// without EXTRA, CLAMP says at compile time whether gamma enters dx clamped (the fused
// LayerNorm's backward does that in both of its modes, the plain one never).
//
// The lean RMSNorm instances (MODE == BWD_RMS without EXTRA) form no column sums of dy: an RMSNorm has no bias, and
// eight additions and eight registers per row and thread are a tenth of the loop.  A caller that asks for dbeta
// under RMSNorm all the same (the dropout-add-norm interface allows it) is served by the general instance.
//
// LEVELS (FIXED instances without optional operands only): the rows lie on several levels (see LevelSteps).  The
// loads are issued in strictly increasing row order, one grid size apart, so the walk index of the next row to
// issue is kept as a running (j0, j1, j2) in scalar registers and advanced by the split grid size with two
// carries: no division in the loop, nothing on the vector unit.  The general instance takes levels too, with
// optional operands, by splitting each row number with two divisions.
template <typename T, int NV, int MODE, int PF, bool EXACT, bool STATS_F32, bool EXTRA, int MAXT, bool FIXED,
          bool CLAMP, bool LEVELS = false>
__global__ __launch_bounds__(MAXT)
void norm_bwd_kernel(NormBwdArgs a) {
  static_assert(!LEVELS || (FIXED && !EXTRA && EXACT), "the running walk index is built for the lean instances");
  constexpr int VEC = VecIO<T>::N;
  constexpr int NE = NV * VEC;
  constexpr int KS = (MODE == BWD_RMS) ? 1 : 2;   // row sums to reduce: RMSNorm has no mean term
  constexpr bool WITH_DB = EXTRA || MODE != BWD_RMS;   // column sums of dy (dbeta)
  using StatT = typename std::conditional<STATS_F32, float, T>::type;
  using RowSums = SumTuple<KS>;
  extern __shared__ float lds[];            // [rows_per_block, cols] column-sum staging
  __shared__ __align__(16) float red[2][kMaxWaves * KS];  // double-buffered by step parity

  const int tpr = FIXED ? MAXT : a.tpr;    // multiple of 64: a wavefront never straddles two rows
  const int rpb = FIXED ? 1 : int(blockDim.x) / tpr;
  const int group = FIXED ? 0 : __builtin_amdgcn_readfirstlane(int(threadIdx.x) / tpr);
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
  [[maybe_unused]] const bool clamp = MODE == BWD_LN_MEMEFF || CLAMP || (EXTRA && a.clamp_gamma != 0);

  float dg[NE], db[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) { dg[e] = 0.f; db[e] = 0.f; }

  const int64_t stride = int64_t(gridDim.x) * rpb;
  const int64_t last_row = a.rows - 1;
  u32x4 nx[PF][NV], ndy[PF][NV];
  StatT nmu[PF], nsv[PF];
  const StatT* meanp = static_cast<const StatT*>(a.mean);
  const StatT* statp = static_cast<const StatT*>(a.stat);
  // LEVELS: walk index of the next row to issue, and where each slot's dx row goes
  [[maybe_unused]] uint32_t wj0 = 0, wj1 = 0, wj2 = 0;
  [[maybe_unused]] int64_t dxo[PF];
  if constexpr (LEVELS) {
    const RowSplit first = split_row(int64_t(blockIdx.x), a.n0, a.n1);
    wj0 = __builtin_amdgcn_readfirstlane(first.j0);
    wj1 = __builtin_amdgcn_readfirstlane(first.j1);
    wj2 = __builtin_amdgcn_readfirstlane(first.j2);
  }
  // loads of row r into slot d; r past the end re-reads the last row (its results are never used)
  auto issue = [&](auto slot, int64_t r) {
    constexpr int d = decltype(slot)::value;
    const int64_t rc = r < last_row ? r : last_row;
    int64_t xo = rc * a.x_pitch, dyo = rc * a.dy_pitch, number = rc;
    if constexpr (LEVELS) {
      // a row past the end reads row 0 instead (any row will do)
      const bool ok = r <= last_row;
      const RowSplit sp{ok ? wj0 : 0u, ok ? wj1 : 0u, ok ? wj2 : 0u};
      xo = split_offset(sp, a.x_pitch, a.x_lv);
      dyo = split_offset(sp, a.dy_pitch, a.dy_lv);
      number = split_number(sp, a.rn);
      dxo[d] = split_offset(sp, a.dx_pitch, a.dx_lv);
      // the next row to issue lies one grid size further on
      wj0 += a.ws0;
      uint32_t carry = wj0 >= uint32_t(a.n0) ? 1u : 0u;
      wj0 -= carry ? uint32_t(a.n0) : 0u;
      wj1 += a.ws1 + carry;
      carry = wj1 >= uint32_t(a.n1) ? 1u : 0u;
      wj1 -= carry ? uint32_t(a.n1) : 0u;
      wj2 += a.ws2 + carry;
    }
    if constexpr (EXTRA) {
      if (a.n0 != a.rows) {   // rows on several levels: uniform
        const RowSplit sp = split_row(rc, a.n0, a.n1);
        xo = split_offset(sp, a.x_pitch, a.x_lv);
        dyo = split_offset(sp, a.dy_pitch, a.dy_lv);
        number = split_number(sp, a.rn);
      }
    }
    if constexpr (MODE == BWD_LN) nmu[d] = meanp[number];
    nsv[d] = statp[number];
    const T* xr = static_cast<const T*>(a.x) + xo;
    const T* dyr = static_cast<const T*>(a.dy) + dyo;
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
    // RMSNorm keeps the inverse root mean square, never a variance
    const float rs = (MODE != BWD_RMS && a.stat_kind == HK_STAT_VAR) ? 1.0f / sqrtf(sv + a.eps) : sv;
    [[maybe_unused]] int64_t dx_offset = 0;
    if constexpr (LEVELS) dx_offset = dxo[d];   // the refill below reuses the slot
    // the slot is free again: refill it with the row PF steps ahead
    issue(slot, row + int64_t(PF) * stride);

    RowSums s = RowSums::identity();
    float& s_prod = s.v[KS - 1];            // sum(dy g xc) (sum(dy (y - beta)) in the memory-efficient mode)
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
          s_prod = fmaf(dz, yb, s_prod);
          dg[e] = fmaf(dz, xhat, dg[e]);
          if constexpr (WITH_DB) db[e] += dz;
          xs[e] = xhat;
          ts[e] = dz * kg;
        } else {
          const float xc = (MODE == BWD_RMS) ? xs[e] : xs[e] - mu;
          const float dzr = dz * rs;
          const float q = dzr * gm[e];
          s_prod = fmaf(q, xc, s_prod);
          if constexpr (MODE != BWD_RMS) s.v[0] += q;
          dg[e] = fmaf(dzr, xc, dg[e]);
          if constexpr (WITH_DB) db[e] += dz;
          xs[e] = xc;
          // the per-element term of dx uses the clamped gamma when asked to
          if constexpr (decltype(clamped)::value) ts[e] = dzr * clamp_by_magnitude(gm[e], a.eps);
          else ts[e] = q;
        }
      }
    };
    if constexpr (!EXTRA) accumulate(std::integral_constant<bool, MODE == BWD_LN_MEMEFF || CLAMP>{});
    else if (clamp) accumulate(std::true_type{});   // uniform
    else accumulate(std::false_type{});

    if constexpr (FIXED) s = group_allreduce_tuple_fixed<RowSums, MAXT / 64>(s, red[parity]);
    else s = group_allreduce_tuple(s, red[parity], first_wave, waves_per_group);
    parity ^= 1;
    if (valid) {
      // plain modes: s0 = rs * sum(dy g), s1 = rs * sum(dy g xc);  dx = q - s0/n - xc * rs^2 * s1/n
      // memory-efficient: s0 = sum(dy g), s1 = sum(dy (y - beta));   dx = rs * (dy kg - s0/n - xhat * s1/n)
      float rc1, k3;
      if constexpr (MODE == BWD_LN_MEMEFF) {
        rc1 = rs * s.v[0] * a.inv_cols;
        k3 = rs * s_prod * a.inv_cols;
      } else {
        rc1 = (MODE == BWD_RMS) ? 0.f : s.v[0] * a.inv_cols;
        k3 = rs * rs * s_prod * a.inv_cols;
      }
      T* dxr = static_cast<T*>(a.dx) + (LEVELS ? dx_offset : row * a.dx_pitch);
      [[maybe_unused]] T* drr = nullptr;
      [[maybe_unused]] const T* dir = nullptr;
      if constexpr (EXTRA) {
        const bool levels = a.n0 != a.rows;   // uniform
        RowSplit sp{};
        if (levels) {
          sp = split_row(row, a.n0, a.n1);
          dxr = static_cast<T*>(a.dx) + split_offset(sp, a.dx_pitch, a.dx_lv);
        }
        if (a.dres) drr = static_cast<T*>(a.dres) + (levels ? split_offset(sp, a.dres_pitch, a.dres_lv) : row * a.dres_pitch);
        if (a.dx_in) {
          dir = static_cast<const T*>(a.dx_in) + (levels ? split_offset(sp, a.dxin_pitch, a.dxin_lv) : row * a.dxin_pitch);
        }
      }
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
          if constexpr (EXTRA) {
            if (dir) {
              float u[VEC];
              VecIO<T>::unpack(ld16(dir + v * VEC), u);
#pragma unroll
              for (int j = 0; j < VEC; ++j) o[j] += u[j];
            }
          }
          const u32x4 pk = VecIO<T>::pack(o);
          st16_stream(dxr + v * VEC, pk);
          if constexpr (EXTRA) {
            if (drr) st16(drr + v * VEC, pk);
          }
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
  if constexpr (FIXED) {
    // one group: every thread writes its own sums, as 16-byte streaming stores (the partial rows are read by the
    // fold kernel, never again by this one; left in the cache they would only wait for the write-back at the
    // kernel's end)
    static_assert(VEC % 4 == 0, "whole float4 vectors per 16-byte vector of the data type");
#pragma unroll
    for (int which = 0; which < (WITH_DB ? 2 : 1); ++which) {
      if (outs[which] == nullptr) continue;
      const float* acc = which == 0 ? dg : db;
      float* dst = outs[which] + int64_t(blockIdx.x) * a.cols;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
#pragma unroll
        for (int j = 0; j < VEC; j += 4) {
          const u32x4 pk = {f2u(acc[i * VEC + j]), f2u(acc[i * VEC + j + 1]), f2u(acc[i * VEC + j + 2]),
                            f2u(acc[i * VEC + j + 3])};
          st16_stream(dst + vidx[i] * VEC + j, pk);
        }
      }
    }
    return;
  }
#pragma unroll
  for (int which = 0; which < (WITH_DB ? 2 : 1); ++which) {
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
  const int64_t i0 = blockIdx.x;                       // row within the innermost level
  const int64_t row = dense_row_index(i0, a.rn);
  const T* xr = static_cast<const T*>(a.x) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
  const T* dyr = static_cast<const T*>(a.dy) + i0 * a.dy_pitch + outer_level_offset(a.dy_lv);
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
  T* dxr = static_cast<T*>(a.dx) + i0 * a.dx_pitch + outer_level_offset(a.dx_lv);
  T* drr = a.dres ? static_cast<T*>(a.dres) + i0 * a.dres_pitch + outer_level_offset(a.dres_lv) : nullptr;
  const T* dir = a.dx_in ? static_cast<const T*>(a.dx_in) + i0 * a.dxin_pitch + outer_level_offset(a.dxin_lv) : nullptr;
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
    const bool levels = a.n0 != a.rows;
    for (int64_t r = w; r < a.rows; r += 4) {
      int64_t dyo = r * a.dy_pitch, xo = r * a.x_pitch, number = r;
      if (levels) {
        const RowSplit sp = split_row(r, a.n0, a.n1);
        dyo = split_offset(sp, a.dy_pitch, a.dy_lv);
        xo = split_offset(sp, a.x_pitch, a.x_lv);
        number = split_number(sp, a.rn);
      }
      const CT d = GenericIO<T, CT>::ld(static_cast<const T*>(a.dy) + dyo + c);
      const CT xv = GenericIO<T, CT>::ld(static_cast<const T*>(a.x) + xo + c);
      CT xhat;
      if (mode == BWD_LN_MEMEFF) {
        xhat = (xv - b) / kg;
      } else {
        const CT sv = a.stats_f32 ? CT(static_cast<const float*>(a.stat)[number])
                                  : GenericIO<T, CT>::ld(static_cast<const T*>(a.stat) + number);
        const CT rs = a.stat_kind == HK_STAT_VAR ? CT(1) / sqrt(sv + CT(a.eps)) : sv;
        CT mu = 0;
        if (mode == BWD_LN)
          mu = a.stats_f32 ? CT(static_cast<const float*>(a.mean)[number])
                           : GenericIO<T, CT>::ld(static_cast<const T*>(a.mean) + number);
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

template <typename T>
BwdPlan plan_norm_bwd(int64_t rows, int cols, bool aligned) {
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

// launch bound of the kernel instance that runs a block of `block` threads
static inline int bound_for(int block) {
  return block <= 512 ? 512 : (block <= 640 ? 640 : (block <= 768 ? 768 : 1024));
}

template <typename T, int MODE, int NV, int MAXT>
static int launch_norm_bwd_inst(const NormBwdArgs& a, const BwdPlan& p, int pf, hipStream_t s) {
  dim3 grid{unsigned(p.grid)}, block{unsigned(p.block)};
  const bool exact = int64_t(p.nv) * p.tpr == a.nvec;
  const bool f32 = a.stats_f32 != 0;
  // the kernel's "extra" instance takes the optional operands behind uniform branches, and the clamp request in
  // the modes that have no instance of their own for it
  const bool want_clamp = a.clamp_gamma != 0 && MODE != BWD_LN_MEMEFF;   // the memory-efficient mode always clamps
  // one group that is the whole block, of exactly the bound's size: the instance with a constant group width
  const bool fixed = p.rpb == 1 && p.block == MAXT;
  // rows on several levels: the lean fixed instances keep a running walk index; every other case splits each row
  // number in the general instance
  const bool levels = a.n0 != a.rows;
  // (dbeta under RMSNorm counts as optional: the lean RMSNorm instances do not form it)
  const bool optional = a.dx_in != nullptr || a.dres != nullptr || (want_clamp && MODE != BWD_LN) ||
                        (MODE == BWD_RMS && a.part_dbeta != nullptr);
  const bool extra = optional || (levels && !(fixed && exact));
  // the deep ring exists for the plain case only: full rows, no optional operands
  if (!exact || extra) pf = 1;
#define HK_BWD_LAUNCH_L(P, E, F, X, FX, C, L) \
  HK_LAUNCH((norm_bwd_kernel<T, NV, MODE, P, E, F, X, MAXT, FX, C, L>), grid, block, p.lds_bytes, s, a)
#define HK_BWD_LAUNCH(P, E, F, X, FX, C) HK_BWD_LAUNCH_L(P, E, F, X, FX, C, false)
#define HK_BWD_LEAN_L(P, F, FX, L)                                          \
  do {                                                                      \
    if constexpr (MODE == BWD_LN) {                                         \
      if (want_clamp) HK_BWD_LAUNCH_L(P, true, F, false, FX, true, L); else HK_BWD_LAUNCH_L(P, true, F, false, FX, false, L); \
    } else {                                                                \
      HK_BWD_LAUNCH_L(P, true, F, false, FX, false, L);                     \
    }                                                                       \
  } while (0)
#define HK_BWD_LEAN(P, F, FX) HK_BWD_LEAN_L(P, F, FX, false)
#define HK_BWD_F(F)                                                         \
  do {                                                                      \
    if (exact && !extra && fixed && levels) { if (pf >= 2) HK_BWD_LEAN_L(2, F, true, true); else HK_BWD_LEAN_L(1, F, true, true); } \
    else if (exact && !extra && fixed) { if (pf >= 2) HK_BWD_LEAN(2, F, true); else HK_BWD_LEAN(1, F, true); } \
    else if (exact && !extra) { if (pf >= 2) HK_BWD_LEAN(2, F, false); else HK_BWD_LEAN(1, F, false); } \
    else if (exact) HK_BWD_LAUNCH(1, true, F, true, false, false);          \
    else if (!extra && !want_clamp) HK_BWD_LAUNCH(1, false, F, false, false, false); \
    else HK_BWD_LAUNCH(1, false, F, true, false, false);                    \
  } while (0)
  if constexpr (MODE == BWD_LN && !std::is_same<T, float>::value) {
    if (f32) HK_BWD_F(true); else HK_BWD_F(false);
  } else {
    HK_BWD_F(true);   // for float data "statistics in the data type" and "in float" are the same kernel
  }
#undef HK_BWD_F
#undef HK_BWD_LEAN
#undef HK_BWD_LEAN_L
#undef HK_BWD_LAUNCH
#undef HK_BWD_LAUNCH_L
  return HK_OK;
}

template <typename T, int MODE>
static int launch_norm_bwd_nv(const NormBwdArgs& a, const BwdPlan& p, hipStream_t s) {
  int pf = tune_get(TUNE_NORM_BWD_PREFETCH);
  // Rows in flight per thread group, measured on the lean instances: at 512 threads per row (4096 bf16 columns,
  // RMSNorm, main kernel) depth 1 / 2 / 3 / 4 / 6 run 134.8 / 130.4 / 133.0 / 134.0 / 136.5 us; at 640 threads
  // (5120 columns, LayerNorm) depth 1 / 2 / 3 run 85.2 / 85.7 / 87.6 us and depths 4 and 6 collapse (252 / 371 us).
  // More bytes in flight than two rows of a 512-thread group (32 KB per compute unit) only lose, as they do for a
  // plain copy kernel; deeper instances than 2 are therefore not built.
  if (pf <= 0) pf = p.block <= 512 ? 2 : 1;
  // statistics in the data dtype only ever come with the plain LayerNorm backward
  if (!a.stats_f32 && MODE != BWD_LN) {
    set_last_error("norm_bwd: this mode keeps its statistics in float32");
    return HK_ERR_INVALID;
  }
  const int bound = bound_for(p.block);
  const bool have_kernel = p.nv == 1 || p.nv == 2 || (p.nv == 4 && VecIO<T>::N == 4);
  if (!have_kernel) {
    set_last_error("norm_bwd: no kernel for %d vectors per thread", p.nv);
    return HK_ERR_UNSUPPORTED;
  }
  // every argument check has passed: only now are the timing events of a measurement handed to the launch, so an
  // early return never leaves them for an unrelated launch to claim
  profile_before(s);
  int rc = HK_ERR_UNSUPPORTED;
  if (p.nv == 1) {
    if (bound == 512) rc = launch_norm_bwd_inst<T, MODE, 1, 512>(a, p, pf, s);
    else if (bound == 640) rc = launch_norm_bwd_inst<T, MODE, 1, 640>(a, p, pf, s);
    else if (bound == 768) rc = launch_norm_bwd_inst<T, MODE, 1, 768>(a, p, pf, s);
    else rc = launch_norm_bwd_inst<T, MODE, 1, 1024>(a, p, pf, s);
  } else if (p.nv == 2) {
    rc = launch_norm_bwd_inst<T, MODE, 2, 512>(a, p, pf, s);       // plans with nv > 1 stay within 512 threads
  } else if (p.nv == 4) {
    if constexpr (VecIO<T>::N == 4) rc = launch_norm_bwd_inst<T, MODE, 4, 512>(a, p, pf, s);
  }
  profile_after(s);
  if (rc != HK_OK) return rc;
  return launch_check("norm_bwd_kernel");
}

template <typename T>
int norm_bwd_typed(NormBwdArgs a, int mode, void* dgamma, void* dbeta, void* ws, size_t ws_bytes,
                   hipStream_t s) {
  constexpr int VEC = VecIO<T>::N;
  auto steps_ok = [](int64_t pitch, const LevelSteps& l) { return pitch % VEC == 0 && l.p1 % VEC == 0 && l.p2 % VEC == 0; };
  const bool aligned = aligned16(a.dy) && aligned16(a.x) && aligned16(a.dx) && aligned16(a.gamma) &&
                       aligned16(a.beta) && aligned16(a.dx_in) && aligned16(a.dres) &&
                       steps_ok(a.dy_pitch, a.dy_lv) && steps_ok(a.x_pitch, a.x_lv) && steps_ok(a.dx_pitch, a.dx_lv) &&
                       (!a.dx_in || steps_ok(a.dxin_pitch, a.dxin_lv)) && (!a.dres || steps_ok(a.dres_pitch, a.dres_lv));
  BwdPlan p = plan_norm_bwd<T>(a.rows, a.cols, aligned);
  if (!p.reg_path) {
    HK_LAUNCH((norm_bwd_generic_dx_kernel<T, float>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)), dim3(256),
              0, s, a, mode);
    int rc = launch_check("norm_bwd_generic_dx_kernel");
    if (rc != HK_OK) return rc;
    if (dgamma || dbeta) {
      HK_LAUNCH((norm_bwd_generic_cols_kernel<T, float>), dim3(unsigned((a.cols + 63) / 64)),
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
  {
    // the walking kernel's row stride, split over the walk levels (used by the instances with a running walk index)
    const uint64_t stride = uint64_t(p.grid) * uint64_t(p.rpb);
    const uint64_t q = stride / uint64_t(a.n0);
    a.ws0 = uint32_t(stride - q * uint64_t(a.n0));
    a.ws1 = uint32_t(q % uint64_t(a.n1));
    a.ws2 = uint32_t(q / uint64_t(a.n1));
  }
  int rc;
  switch (mode) {
    case BWD_LN: rc = launch_norm_bwd_nv<T, BWD_LN>(a, p, s); break;
    case BWD_RMS: rc = launch_norm_bwd_nv<T, BWD_RMS>(a, p, s); break;
    default: rc = launch_norm_bwd_nv<T, BWD_LN_MEMEFF>(a, p, s); break;
  }
  if (rc != HK_OK || !want_cols) return rc;
  HK_LAUNCH((norm_bwd_finalize_kernel<T>), dim3(unsigned((a.cols + 127) / 128), 2), dim3(512), 0, s,
                     a.part_dgamma, a.part_dbeta, static_cast<T*>(dgamma), static_cast<T*>(dbeta),
                     p.grid, a.cols);
  return launch_check("norm_bwd_finalize_kernel");
}

} // namespace hk
