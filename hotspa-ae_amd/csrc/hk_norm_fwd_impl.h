// LayerNorm / RMSNorm forward kernels and their launch logic, included by the per-type instantiation files.
//
// A row is read once with 128-bit loads and lives in fp32 registers; its sums are reduced across lanes (DPP) and
// wavefronts (LDS), the output is written with 128-bit stores.  One wavefront per row for short rows, one
// workgroup per row for long rows.
#pragma once

#include "hk_norm.h"

namespace hk {

// T: element type; NV: 16-byte vectors per thread and row; WAVE_ROW: one wavefront per row (4 rows per 256-thread
// block) instead of one workgroup per row; HAS_RES: x = x0 + residual is formed in fp32 and optionally written
// back; IS_RMS: RMSNorm (no centring, no bias term in the statistics); R: rows a workgroup takes, 1 or 2.
//
// With R > 1 a thread holds its columns of R consecutive rows: all their loads are issued back to back, each
// reduction carries every row's sums through one barrier, and gamma / beta are fetched once for the lot.  The
// parameter fetches go through the compute unit's vector cache like the rows themselves and are as many bytes per
// row as the row: with gamma and beta a one-row workgroup moves three rows' worth through that cache for every
// row it reads, and the kernel pays for it (4096 bf16 columns, 32768 rows: 86 us with gamma alone, 92 us with
// gamma and beta).
//
// Every row operand is addressed through a buffer descriptor of exactly one row (base = the row's first byte,
// size = cols * sizeof(T)): the hardware returns zeros for a lane past the row's end and drops its stores, so no
// memory instruction sits inside a branch and all of a thread's loads are issued back to back.  The second row of
// the last workgroup of an odd number of rows gets an empty descriptor in the same way.
//
// A row is unpacked to fp32 registers once and, for LayerNorm, centred in place by the second statistics pass, so
// the normalisation costs one multiply and one multiply-add per element.  Which values stay in registers across
// the reductions is written out here rather than left to the compiler: with the row kept packed and unpacked again
// per pass, unrelated edits moved the 5120-column bf16 kernel between 57.7 and 61 us.
template <typename T, int NV, bool WAVE_ROW, bool HAS_RES, bool IS_RMS, int R>
__global__ __launch_bounds__(WAVE_ROW ? 256 : (R >= 2 ? 512 : 1024))   // several rows: at most 512 threads
void norm_fwd_kernel(NormFwdArgs a) {
  static_assert(R == 1 || !WAVE_ROW, "a wavefront takes one row");
  constexpr int VEC = VecIO<T>::N;
  constexpr int NE = NV * VEC;
  __shared__ __align__(16) float red[2][kMaxWaves * 2 * R];   // one slot per reduction of the kernel

  const int tpr = WAVE_ROW ? kWave : int(blockDim.x);
  const int t = WAVE_ROW ? int(threadIdx.x & 63) : int(threadIdx.x);
  const int64_t row0 = WAVE_ROW
      ? int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_index()
      : int64_t(blockIdx.x) * R;
  // row0 counts along the first walk level; blockIdx.y / z are the other two (one level: both 0)
  if (WAVE_ROW && row0 >= a.n0) return;  // wave-uniform; no block barrier in this mode
  const int nwaves = WAVE_ROW ? 1 : int(blockDim.x >> 6);
  auto off = [&](int i) { return uint32_t(i * tpr + t) * 16u; };   // vector i of thread t, in bytes from the row's start
  // long rows: stops the scheduler from unpacking every vector of a pass before the first one is consumed
  auto fence = [] { if constexpr (NV * R >= 8) __builtin_amdgcn_sched_barrier(0); };

  // row r of this workgroup; one past the end is addressed as the first row with a size of zero bytes
  int64_t rowi[R];
  uint32_t bytes[R];
  bool live[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    live[r] = r == 0 || row0 + r < a.n0;
    rowi[r] = live[r] ? row0 + r : row0;
    bytes[r] = live[r] ? uint32_t(a.nvec) * 16u : 0u;
  }

  float v[R][NE];
  {
    u32x4 raw[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const BufferRsrc xr = make_rsrc(static_cast<const T*>(a.x) + rowi[r] * a.x_pitch + outer_level_offset(a.x_lv),
                                      bytes[r]);
#pragma unroll
      for (int i = 0; i < NV; ++i) raw[r][i] = buf_ld16<kBufStream>(xr, off(i));
    }
    if constexpr (HAS_RES) {
      u32x4 res[R][NV];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const BufferRsrc rr = make_rsrc(static_cast<const T*>(a.residual) + rowi[r] * a.res_pitch +
                                        outer_level_offset(a.res_lv), bytes[r]);
#pragma unroll
        for (int i = 0; i < NV; ++i) res[r][i] = buf_ld16<kBufStream>(rr, off(i));
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        // an absent x_out becomes an empty buffer: its stores are dropped by the bounds check
        const BufferRsrc xo = make_rsrc(a.x_out ? static_cast<T*>(a.x_out) + rowi[r] * a.xout_pitch +
                                                      outer_level_offset(a.xout_lv)
                                                : static_cast<T*>(a.y), a.x_out ? bytes[r] : 0u);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          float f1[VEC];
          VecIO<T>::unpack(raw[r][i], &v[r][i * VEC]);
          VecIO<T>::unpack(res[r][i], f1);
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[r][i * VEC + j] += f1[j];
          buf_st16<kBufStream>(xo, off(i), VecIO<T>::pack(&v[r][i * VEC]));
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = 0; i < NV; ++i) { fence(); VecIO<T>::unpack(raw[r][i], &v[r][i * VEC]); }
      }
    }
  }

  // sums over the group of threads that holds the rows; the two reductions of a kernel use separate LDS slots,
  // so no barrier is needed between them
  auto allred = [&](auto s, int slot) {
    if constexpr (WAVE_ROW) return wave_allreduce_tuple(s);
    else return group_allreduce_tuple(s, red[slot], 0, nwaves);
  };

  float mu[R], rs[R], var[R];
  if constexpr (IS_RMS) {
    // lanes past the row's end hold zeros, which add nothing to either sum; one reduction carries both sums
    SumTuple<2 * R> both;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s0 = 0.f, ss = 0.f;
#pragma unroll
      for (int e = 0; e < NE; ++e) { s0 += v[r][e]; ss = fmaf(v[r][e], v[r][e], ss); }
      both.v[2 * r] = ss;
      both.v[2 * r + 1] = s0;
    }
    both = allred(both, 0);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float ms = both.v[2 * r] * a.inv_cols;   // mean(x^2) = var + mu^2
      mu[r] = both.v[2 * r + 1] * a.inv_cols;
      var[r] = fmaxf(ms - mu[r] * mu[r], 0.f);
      rs[r] = 1.0f / sqrtf(ms + a.eps);
    }
  } else {
    // Two passes over the registers: the mean first, then the sum of squares about it, each reduced over the
    // group.  Centring on the row's own mean keeps fp32 accuracy for rows with an outlier, a large common offset
    // or no variance at all.  The centred values replace the row in the registers.
    SumTuple<R> s1, s2;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < NE; ++e) s += v[r][e];         // zeros past the end
      s1.v[r] = s;
    }
    s1 = allred(s1, 0);
#pragma unroll
    for (int r = 0; r < R; ++r) mu[r] = s1.v[r] * a.inv_cols;
    if (a.nvec == NV * tpr) {                            // uniform: a row fills every lane's every vector
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float m2 = 0.f;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
          v[r][e] -= mu[r];
          m2 = fmaf(v[r][e], v[r][e], m2);
        }
        s2.v[r] = m2;
      }
    } else {
      // a lane past the row's end holds -mu, not data: its vectors are left out.  Kept apart from the full-row
      // case, whose straight-line code the per-vector selects would break up (57.8 against 61 us at 5120 bf16
      // columns).
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float m2 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          float q = 0.f;
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            v[r][i * VEC + j] -= mu[r];
            q = fmaf(v[r][i * VEC + j], v[r][i * VEC + j], q);
          }
          m2 += (i * tpr + t < a.nvec) ? q : 0.f;
        }
        s2.v[r] = m2;
      }
    }
    s2 = allred(s2, 1);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      var[r] = s2.v[r] * a.inv_cols;
      rs[r] = 1.0f / sqrtf(var[r] + a.eps);
    }
  }

  if (t == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (live[r]) {
        const int64_t dense = dense_row_index(rowi[r], a.rn);
        store_stat<T>(a.mean, dense, mu[r], a.stats_f32);
        store_stat<T>(a.stat, dense, a.stat_kind == HK_STAT_VAR ? var[r] : rs[r], a.stats_f32);
      }
    }
  }

  BufferRsrc yr[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    yr[r] = make_rsrc(static_cast<T*>(a.y) + rowi[r] * a.y_pitch + outer_level_offset(a.y_lv), bytes[r]);
  const uint32_t row_bytes = uint32_t(a.nvec) * 16u;
  // gamma / beta are fetched after the reduction: every fetch holds one of the compute unit's outstanding-request
  // slots until the data is back; issued before the row has arrived they would hold those slots for the whole HBM
  // latency instead of the L2's.  The four cases of missing parameters are separate straight-line copies, so that
  // no fetch sits inside a branch.
  auto epilogue = [&](auto has_g, auto has_b) {
    constexpr bool HG = decltype(has_g)::value, HB = decltype(has_b)::value;
    const BufferRsrc gr = make_rsrc(HG ? a.gamma : a.y, row_bytes);   // an absent parameter is not fetched at all
    const BufferRsrc br = make_rsrc(HB ? a.beta : a.y, row_bytes);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      [[maybe_unused]] float g[VEC], b[VEC];
      if constexpr (HG) VecIO<T>::unpack(buf_ld16<kBufKeep>(gr, off(i)), g);
      if constexpr (HB) VecIO<T>::unpack(buf_ld16<kBufKeep>(br, off(i)), b);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float f[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float n = rs[r] * v[r][i * VEC + j];
          f[j] = HG ? (HB ? fmaf(g[j], n, b[j]) : g[j] * n) : (HB ? n + b[j] : n);
        }
        buf_st16<kBufStream>(yr[r], off(i), VecIO<T>::pack(f));
      }
      // long rows: keep the compiler from hoisting every parameter fetch above the first store, which would
      // hold 2 * NV more vectors in registers than the row itself
      fence();
    }
  };
  if (a.gamma && a.beta) epilogue(std::true_type{}, std::true_type{});
  else if (a.gamma) epilogue(std::true_type{}, std::false_type{});
  else if (a.beta) epilogue(std::false_type{}, std::true_type{});
  else epilogue(std::false_type{}, std::false_type{});
}

// Fallback for rows that are not a whole number of 16-byte vectors, are not
// 16-byte aligned, or do not fit the register file: one workgroup per row,
// three strided passes (the re-reads hit L2).  CT is the arithmetic type.
template <typename T, typename CT>
__global__ __launch_bounds__(256)
void norm_fwd_generic_kernel(NormFwdArgs a) {
  __shared__ CT lds[256];
  const int64_t i0 = blockIdx.x;                       // row within the innermost level
  const int64_t row = dense_row_index(i0, a.rn);
  const T* xr = static_cast<const T*>(a.x) + i0 * a.x_pitch + outer_level_offset(a.x_lv);
  const T* rr = a.residual ? static_cast<const T*>(a.residual) + i0 * a.res_pitch + outer_level_offset(a.res_lv)
                           : nullptr;
  T* xo = a.x_out ? static_cast<T*>(a.x_out) + i0 * a.xout_pitch + outer_level_offset(a.xout_lv) : nullptr;
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
  T* yr = static_cast<T*>(a.y) + i0 * a.y_pitch + outer_level_offset(a.y_lv);
  const T* gp = static_cast<const T*>(a.gamma);
  const T* bp = static_cast<const T*>(a.beta);
  for (int c = threadIdx.x; c < a.cols; c += blockDim.x) {
    const CT g = gp ? GenericIO<T, CT>::ld(gp + c) : CT(1);
    const CT b = bp ? GenericIO<T, CT>::ld(bp + c) : CT(0);
    GenericIO<T, CT>::st(yr + c, g * (rs * (ldx(c) - shift)) + b);
  }
}

// the most rows a workgroup of the register kernel may take: two where both stay within 80 fp32 registers per
// thread (64 with a residual row in flight next to each).  Four were measured too: 4096 bf16 columns 88.9 us
// against 84.7 us for two and 86.2 us for one, 4096 fp32 columns 45.4 / 45.8 / 46.4 us.
template <typename T>
static constexpr int max_rows_per_block(int nv, bool has_res) {
  const int floats = nv * VecIO<T>::N, budget = has_res ? 64 : 80;
  return floats * 2 <= budget ? 2 : 1;
}

// rows_per_block: 1 or 2 (one-wavefront rows always 1)
template <typename T, int NV, bool WAVE_ROW, bool HAS_RES, bool IS_RMS>
static int launch_norm_fwd_width(const NormFwdArgs& a, int rows_per_block, dim3 grid, dim3 block, hipStream_t s) {
  if constexpr (!WAVE_ROW && max_rows_per_block<T>(NV, HAS_RES) >= 2) {
    if (rows_per_block == 2) {
      // two rows of several vectors per thread: fewer workgroups per compute unit than the thread limit admits
      // stream faster (256 threads: 5 instead of 8, 83.5 against 84.8 us at 4096 bf16 columns; 512 threads: 3
      // instead of 4, 44.7 against 45.9 us at 4096 fp32 columns; 2 lose again)
      int resident = tune_get(TUNE_NORM_FWD_RESIDENT);
      if (resident == 0) resident = block.x == 256 ? 5 : (block.x == 512 ? 3 : 0);
      size_t lds = 0;
      HK_REQUIRE(lds_bytes_for_residency(resident, sizeof(float) * 2 * kMaxWaves * 2 * 2, &lds), HK_ERR_INVALID,
                 "norm_fwd: 'norm_fwd_resident' = %d needs more dynamic LDS than one workgroup may ask for", resident);
      profile_before(s);
      HK_LAUNCH((norm_fwd_kernel<T, NV, false, HAS_RES, IS_RMS, 2>), grid, block, lds, s, a);
      profile_after(s);
      return HK_OK;
    }
  }
  profile_before(s);
  HK_LAUNCH((norm_fwd_kernel<T, NV, WAVE_ROW, HAS_RES, IS_RMS, 1>), grid, block, 0, s, a);
  profile_after(s);
  return HK_OK;
}

template <typename T, bool WAVE_ROW, bool HAS_RES, bool IS_RMS>
static int launch_norm_fwd_rms(const NormFwdArgs& a, int nv, int rpb, dim3 grid, dim3 block, hipStream_t s) {
  // the timing events of a measurement are handed to the launch only once every argument check has passed
  // (launch_norm_fwd_width), so an early return never leaves them for an unrelated launch to claim
  int rc = HK_ERR_UNSUPPORTED;
  switch (nv) {
    case 1: rc = launch_norm_fwd_width<T, 1, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 2: rc = launch_norm_fwd_width<T, 2, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 3: rc = launch_norm_fwd_width<T, 3, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 4: rc = launch_norm_fwd_width<T, 4, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 5: rc = launch_norm_fwd_width<T, 5, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 6: rc = launch_norm_fwd_width<T, 6, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 8: rc = launch_norm_fwd_width<T, 8, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s); break;
    case 16:
      // sixteen vectors are 64 fp32 registers only for fp32 data; with a residual two packed rows of that length
      // are in flight on top
      if constexpr (sizeof(T) == 4 && !WAVE_ROW && !HAS_RES) {
        rc = launch_norm_fwd_width<T, 16, WAVE_ROW, HAS_RES, IS_RMS>(a, rpb, grid, block, s);
        break;
      }
      [[fallthrough]];
    default:
      set_last_error("norm_fwd: no kernel for %d vectors per thread", nv);
      return HK_ERR_UNSUPPORTED;
  }
  if (rc != HK_OK) return rc;
  return launch_check("norm_fwd_kernel");
}

template <typename T, bool WAVE_ROW, bool HAS_RES>
static int launch_norm_fwd_nv(const NormFwdArgs& a, int nv, int rpb, dim3 grid, dim3 block, hipStream_t s) {
  return a.is_rms ? launch_norm_fwd_rms<T, WAVE_ROW, HAS_RES, true>(a, nv, rpb, grid, block, s)
                  : launch_norm_fwd_rms<T, WAVE_ROW, HAS_RES, false>(a, nv, rpb, grid, block, s);
}

// Picks threads-per-row and vectors-per-thread for a row of `nvec` 16-byte
// vectors.  Returns false when the row does not fit the register kernels.
static bool pick_row_shape(int nvec, int forced_threads, int max_nv, int wave_row_max_nv, bool many_rows,
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
  // A 512-thread workgroup (two wavefronts on each of the four SIMDs) is as good when it gets by with two vectors
  // (4096 fp32 columns: 46 us against 49 us for 256 x 4); widths that load the SIMDs unevenly (320, 384) are not,
  // except that 320 x 2 beats 128 x 5 once the input is large enough for two rows per workgroup (5120 bf16
  // columns, 16384 rows: 55.4 against 56.4 us; one row per workgroup: 61.4 against 57.7 us).
  static const int kCounts[] = {2, 3, 4, 5, 6, 8};
  for (int n : kCounts) {
    if (n > max_nv) break;
    int t = ((nvec + n - 1) / n + 63) / 64 * 64;
    if ((t <= 256 || (t == 512 && n == 2) || (t == 320 && n == 2 && many_rows)) && n * t == nvec) {
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
int norm_fwd_typed(NormFwdArgs a, hipStream_t s) {
  constexpr int VEC = VecIO<T>::N;
  auto pitch_ok = [](int64_t p) { return p % VEC == 0; };
  auto steps_ok = [](int64_t pitch, const LevelSteps& l) { return pitch % VEC == 0 && l.p1 % VEC == 0 && l.p2 % VEC == 0; };
  (void)pitch_ok;
  const bool vec_ok = (a.cols % VEC == 0) && aligned16(a.x) && aligned16(a.y) &&
                      aligned16(a.gamma) && aligned16(a.beta) && aligned16(a.residual) &&
                      aligned16(a.x_out) && steps_ok(a.x_pitch, a.x_lv) && steps_ok(a.y_pitch, a.y_lv) &&
                      (!a.residual || steps_ok(a.res_pitch, a.res_lv)) &&
                      (!a.x_out || steps_ok(a.xout_pitch, a.xout_lv));
  int threads = 0, nv = 0;
  a.nvec = a.cols / VEC;
  const bool has_res = a.residual != nullptr;
  // the row is held as at most 64 fp32 registers per thread (and at most 8 vectors when a residual row is in
  // flight next to it)
  const int max_nv = has_res ? std::min(8, 64 / VEC) : 64 / VEC;
  const int wave_nv = has_res ? (VEC == 4 ? 8 : 4) : (VEC == 4 ? 16 : 8);
  // large inputs take two rows per workgroup (below), which also changes the best width of some rows
  const int want_rows = tune_get(TUNE_NORM_FWD_ROWS);
  const bool many_rows = want_rows > 0 ? want_rows >= 2 : a.rows >= 16 * int64_t(device_cu_count());
  if (vec_ok &&
      pick_row_shape(a.nvec, tune_get(TUNE_NORM_FWD_THREADS), max_nv, wave_nv, many_rows, &threads, &nv)) {
    if (threads == 64) {
      dim3 grid(unsigned((a.n0 + 3) / 4), unsigned(a.n1), unsigned(a.n2)), block(256);
      return has_res ? launch_norm_fwd_nv<T, true, true>(a, nv, 1, grid, block, s)
                     : launch_norm_fwd_nv<T, true, false>(a, nv, 1, grid, block, s);
    }
    // two rows per workgroup where both fit the registers (the same bound as in launch_norm_fwd_width) and the
    // grid still fills the device many times over
    int rpb = 1;
    if (threads <= 512) {
      const int most = max_rows_per_block<T>(nv, has_res);
      rpb = std::min(many_rows ? 2 : 1, most);
    }
    dim3 grid{unsigned((a.n0 + rpb - 1) / rpb), unsigned(a.n1), unsigned(a.n2)}, block{unsigned(threads)};
    return has_res ? launch_norm_fwd_nv<T, false, true>(a, nv, rpb, grid, block, s)
                   : launch_norm_fwd_nv<T, false, false>(a, nv, rpb, grid, block, s);
  }
  HK_LAUNCH((norm_fwd_generic_kernel<T, float>), dim3(unsigned(a.n0), unsigned(a.n1), unsigned(a.n2)), dim3(256), 0,
            s, a);
  return launch_check("norm_fwd_generic_kernel");
}

} // namespace hk
