// Streaming yardstick: a kernel that only moves bytes, NR arrays read and NW arrays written per launch, in every
// launch shape a row kernel could take (workgroup size, 16-byte vectors in flight per thread, one-shot grid or a
// fixed number of workgroups per compute unit walking the array, non-temporal hint on the loads and / or the
// stores).  What the best shape of a mix reaches is the roof the operator kernels with that mix are held against.
// The hints are template arguments: as run-time flags the compiler merges the two branches into a plain access.
//
// This file is a library of its own (libhk_bench.so, include/hk_bench.h) that bench.py loads: a measurement tool, kept
// out of the operator library.  It shares hk_common.h's device-side types with the kernels and nothing else.
#include "hk_common.h"
#include "hk_bench.h"

#include <algorithm>
#include <stdarg.h>
#include <stdio.h>

namespace hk {

static thread_local char g_bench_error[512] = "";

// this library's own error text (the operator library's is not shared with it)
void set_last_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_bench_error, sizeof(g_bench_error), fmt, ap);
  va_end(ap);
}

static int bench_launch_check(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return HK_OK;
  set_last_error("%s: launch failed: %s", what, hipGetErrorString(e));
  return HK_ERR_HIP;
}

static int bench_cu_count() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
  return n;
}

struct ProbeArgs {
  const u32x4* src[2];
  u32x4* dst[2];
  size_t nvec;
  uint32_t* sink;
};

template <int BS, int U, int NR, int NW, bool NTL, bool NTS>
__global__ __launch_bounds__(BS)
void stream_probe_kernel(ProbeArgs a) {
  const size_t tile = size_t(BS) * U;
  uint32_t acc = 0;
  // grid-stride over tiles of BS * U vectors; a one-shot launch has one tile per workgroup
  for (size_t t0 = size_t(blockIdx.x) * tile; t0 < a.nvec; t0 += size_t(gridDim.x) * tile) {
    const size_t base = t0 + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int i = 0; i < U; ++i) v[i] = u32x4{1u, 2u, 3u, uint32_t(threadIdx.x)};
    if constexpr (NR >= 1) {
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const size_t idx = base + size_t(i) * BS;
        if (idx < a.nvec) v[i] = NTL ? __builtin_nontemporal_load(a.src[0] + idx) : a.src[0][idx];
      }
    }
    if constexpr (NR >= 2) {
      u32x4 w[U];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const size_t idx = base + size_t(i) * BS;
        w[i] = u32x4{0, 0, 0, 0};
        if (idx < a.nvec) w[i] = NTL ? __builtin_nontemporal_load(a.src[1] + idx) : a.src[1][idx];
      }
#pragma unroll
      for (int i = 0; i < U; ++i) v[i] ^= w[i];
    }
#pragma unroll
    for (int o = 0; o < NW; ++o) {
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const size_t idx = base + size_t(i) * BS;
        if (idx < a.nvec) {
          if constexpr (NTS) __builtin_nontemporal_store(v[i], a.dst[o] + idx);
          else a.dst[o][idx] = v[i];
        }
      }
    }
    if constexpr (NW == 0) {
#pragma unroll
      for (int i = 0; i < U; ++i) acc += v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
  }
  if (NW == 0 && acc == 0x12345678u && a.sink) a.sink[0] = acc;   // keeps the loads of a read-only run alive
}

template <int BS, int U, int NR, int NW>
static int probe_nt(const ProbeArgs& a, int ntl, int nts, unsigned grid, hipStream_t s) {
  if (NR == 0) ntl = 0;
  if (NW == 0) nts = 0;
#define HK_PROBE(L, S) hipLaunchKernelGGL((stream_probe_kernel<BS, U, NR, NW, L, S>), dim3(grid), dim3(BS), 0, s, a)
  if (ntl && nts) HK_PROBE(NR != 0, NW != 0);
  else if (ntl) HK_PROBE(NR != 0, false);
  else if (nts) HK_PROBE(false, NW != 0);
  else HK_PROBE(false, false);
#undef HK_PROBE
  return bench_launch_check("stream_probe_kernel");
}

template <int BS, int U>
static int probe_mix(const ProbeArgs& a, int nr, int nw, int ntl, int nts, unsigned grid, hipStream_t s) {
  if (nr == 1 && nw == 1) return probe_nt<BS, U, 1, 1>(a, ntl, nts, grid, s);
  if (nr == 2 && nw == 1) return probe_nt<BS, U, 2, 1>(a, ntl, nts, grid, s);
  if (nr == 1 && nw == 2) return probe_nt<BS, U, 1, 2>(a, ntl, nts, grid, s);
  if (nr == 1 && nw == 0) return probe_nt<BS, U, 1, 0>(a, ntl, nts, grid, s);
  if (nr == 0 && nw == 1) return probe_nt<BS, U, 0, 1>(a, ntl, nts, grid, s);
  set_last_error("hk_bench_stream_probe: no kernel for %d reads : %d writes", nr, nw);
  return HK_ERR_UNSUPPORTED;
}

template <int BS>
static int probe_unroll(const ProbeArgs& a, int unroll, int nr, int nw, int ntl, int nts, unsigned grid, hipStream_t s) {
  switch (unroll) {
    case 1: return probe_mix<BS, 1>(a, nr, nw, ntl, nts, grid, s);
    case 2: return probe_mix<BS, 2>(a, nr, nw, ntl, nts, grid, s);
    case 4: return probe_mix<BS, 4>(a, nr, nw, ntl, nts, grid, s);
    default:
      set_last_error("hk_bench_stream_probe: 1, 2 or 4 vectors per thread, got %d", unroll);
      return HK_ERR_UNSUPPORTED;
  }
}

// The persistent 2R:1W walk once more, software-pipelined the way the backward norm kernels are: a workgroup owns
// every gridDim.x-th tile of BS vectors, keeps a ring of PF tiles of both input arrays in flight per thread (a slot is
// refilled as soon as it has been consumed, loads past the end re-read the last tile), and optionally goes through one
// workgroup barrier with a small LDS exchange per tile, which is what a row reduction across the wavefronts costs.
// What the best depth reaches is the ceiling of that kernel design, whatever arithmetic is put into it.
struct RingArgs {
  const u32x4* a;
  const u32x4* b;
  u32x4* d;
  long ntiles;
};

template <int BS, int PF, bool BARRIER>
__global__ __launch_bounds__(BS)
void ring_probe_kernel(RingArgs p) {
  __shared__ uint32_t red[2][16];
  u32x4 va[PF], vb[PF];
  const long G = gridDim.x;
  const long last = p.ntiles - 1;
  long t0 = blockIdx.x;
  auto issue = [&](auto slot, long t) {
    constexpr int s = decltype(slot)::value;
    const long tc = t < last ? t : last;
    va[s] = __builtin_nontemporal_load(p.a + tc * BS + threadIdx.x);
    vb[s] = __builtin_nontemporal_load(p.b + tc * BS + threadIdx.x);
  };
  static_for<PF>([&](auto slot) { issue(slot, t0 + decltype(slot)::value * G); });
  int parity = 0;
  auto step = [&](auto slot, auto guarded) {
    constexpr int s = decltype(slot)::value;
    const long t = t0 + s * G;
    u32x4 r = va[s] ^ vb[s];
    issue(slot, t + PF * G);
    if constexpr (BARRIER) {
      uint32_t v = r.x + r.y;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) v += uint32_t(__shfl_xor(int(v), o));
      if ((threadIdx.x & 63) == 0) red[parity][threadIdx.x >> 6] = v;
      __syncthreads();
      uint32_t total = 0;
#pragma unroll
      for (int w = 0; w < BS / 64; ++w) total += red[parity][w];
      parity ^= 1;
      r.w ^= total;
    }
    if (!decltype(guarded)::value || t < p.ntiles) __builtin_nontemporal_store(r, p.d + t * BS + threadIdx.x);
  };
  long base = blockIdx.x;
  const long round = long(PF) * G;
#pragma nounroll
  for (; base + long(PF - 1) * G < p.ntiles; base += round) {
    static_for<PF>([&](auto slot) { step(slot, std::false_type{}); });
    t0 += round;
  }
#pragma nounroll
  for (; base < p.ntiles; base += round) {
    static_for<PF>([&](auto slot) { step(slot, std::true_type{}); });
    t0 += round;
  }
}

template <int BS, int PF>
static int ring_barrier(const RingArgs& a, int barrier, unsigned grid, hipStream_t s) {
  if (barrier) hipLaunchKernelGGL((ring_probe_kernel<BS, PF, true>), dim3(grid), dim3(BS), 0, s, a);
  else hipLaunchKernelGGL((ring_probe_kernel<BS, PF, false>), dim3(grid), dim3(BS), 0, s, a);
  return bench_launch_check("ring_probe_kernel");
}

template <int BS>
static int ring_depth(const RingArgs& a, int depth, int barrier, unsigned grid, hipStream_t s) {
  switch (depth) {
    case 1: return ring_barrier<BS, 1>(a, barrier, grid, s);
    case 2: return ring_barrier<BS, 2>(a, barrier, grid, s);
    case 3: return ring_barrier<BS, 3>(a, barrier, grid, s);
    case 4: return ring_barrier<BS, 4>(a, barrier, grid, s);
    default:
      set_last_error("hk_bench_ring_probe: ring depth 1 to 4, got %d", depth);
      return HK_ERR_UNSUPPORTED;
  }
}

} // namespace hk

using namespace hk;

extern "C" {

const char* hk_bench_last_error(void) { return g_bench_error; }

int hk_bench_stream_probe(void* dst0, void* dst1, const void* src0, const void* src1, int reads, int writes,
                          size_t bytes, int block_threads, int vectors_per_thread, int nt_loads, int nt_stores,
                          int workgroups_per_cu, hkStream_t stream) {
  const char* who = "hk_bench_stream_probe";
  HK_REQUIRE(block_threads == 64 || block_threads == 128 || block_threads == 256 || block_threads == 512 ||
             block_threads == 1024, HK_ERR_UNSUPPORTED, "%s: workgroups of 64, 128, 256, 512 or 1024 threads, got %d",
             who, block_threads);
  HK_REQUIRE(vectors_per_thread == 1 || vectors_per_thread == 2 || vectors_per_thread == 4, HK_ERR_UNSUPPORTED,
             "%s: 1, 2 or 4 vectors per thread, got %d", who, vectors_per_thread);
  HK_REQUIRE(bytes % 16 == 0 && bytes > 0, HK_ERR_INVALID, "%s: size must be a positive multiple of 16", who);
  HK_REQUIRE(reads >= 0 && reads <= 2 && writes >= 0 && writes <= 2 && reads + writes > 0, HK_ERR_INVALID,
             "%s: 0..2 reads and 0..2 writes, not both 0", who);
  HK_REQUIRE((reads < 1 || src0) && (reads < 2 || src1) && (writes < 1 || dst0) && (writes < 2 || dst1),
             HK_ERR_INVALID, "%s: null array", who);
  HK_REQUIRE(aligned16(src0) && aligned16(src1) && aligned16(dst0) && aligned16(dst1), HK_ERR_INVALID,
             "%s: arrays must be 16-byte aligned", who);
  HK_REQUIRE(workgroups_per_cu >= 0 && workgroups_per_cu <= 64, HK_ERR_INVALID,
             "%s: 0 (one-shot grid) to 64 workgroups per compute unit", who);
  ProbeArgs a{};
  a.src[0] = static_cast<const u32x4*>(src0); a.src[1] = static_cast<const u32x4*>(src1);
  a.dst[0] = static_cast<u32x4*>(dst0); a.dst[1] = static_cast<u32x4*>(dst1);
  a.nvec = bytes / 16;
  a.sink = nullptr;
  const size_t tile = size_t(block_threads) * size_t(vectors_per_thread);
  const size_t tiles = (a.nvec + tile - 1) / tile;
  HK_REQUIRE(tiles <= 0x7fffffffu, HK_ERR_INVALID, "%s: size too large", who);
  const unsigned grid = workgroups_per_cu == 0 ? unsigned(tiles)
                                               : unsigned(std::min<size_t>(tiles, size_t(bench_cu_count()) * workgroups_per_cu));
  hipStream_t s = as_hip(stream);
  switch (block_threads) {
    case 64: return probe_unroll<64>(a, vectors_per_thread, reads, writes, nt_loads, nt_stores, grid, s);
    case 128: return probe_unroll<128>(a, vectors_per_thread, reads, writes, nt_loads, nt_stores, grid, s);
    case 256: return probe_unroll<256>(a, vectors_per_thread, reads, writes, nt_loads, nt_stores, grid, s);
    case 512: return probe_unroll<512>(a, vectors_per_thread, reads, writes, nt_loads, nt_stores, grid, s);
    default: return probe_unroll<1024>(a, vectors_per_thread, reads, writes, nt_loads, nt_stores, grid, s);
  }
}

int hk_bench_ring_probe(void* dst, const void* src0, const void* src1, size_t bytes, int block_threads, int depth,
                        int barrier, int workgroups_per_cu, hkStream_t stream) {
  const char* who = "hk_bench_ring_probe";
  HK_REQUIRE(block_threads == 256 || block_threads == 512 || block_threads == 1024, HK_ERR_UNSUPPORTED,
             "%s: workgroups of 256, 512 or 1024 threads, got %d", who, block_threads);
  HK_REQUIRE(depth >= 1 && depth <= 4, HK_ERR_UNSUPPORTED, "%s: ring depth 1 to 4, got %d", who, depth);
  HK_REQUIRE(workgroups_per_cu >= 1 && workgroups_per_cu <= 8, HK_ERR_INVALID,
             "%s: 1 to 8 workgroups per compute unit, got %d", who, workgroups_per_cu);
  HK_REQUIRE(dst && src0 && src1, HK_ERR_INVALID, "%s: null array", who);
  HK_REQUIRE(aligned16(dst) && aligned16(src0) && aligned16(src1), HK_ERR_INVALID,
             "%s: arrays must be 16-byte aligned", who);
  const size_t tile_bytes = size_t(block_threads) * 16;
  HK_REQUIRE(bytes > 0 && bytes % tile_bytes == 0, HK_ERR_INVALID,
             "%s: size must be a positive multiple of %zu bytes (whole tiles)", who, tile_bytes);
  RingArgs a{};
  a.a = static_cast<const u32x4*>(src0);
  a.b = static_cast<const u32x4*>(src1);
  a.d = static_cast<u32x4*>(dst);
  a.ntiles = long(bytes / tile_bytes);
  const unsigned grid = unsigned(std::min<size_t>(size_t(a.ntiles), size_t(bench_cu_count()) * workgroups_per_cu));
  hipStream_t s = as_hip(stream);
  switch (block_threads) {
    case 256: return ring_depth<256>(a, depth, barrier, grid, s);
    case 512: return ring_depth<512>(a, depth, barrier, grid, s);
    default: return ring_depth<1024>(a, depth, barrier, grid, s);
  }
}

} // extern "C"
