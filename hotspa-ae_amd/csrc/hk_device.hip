// Device / memory / stream / event entry points of the C-ABI, plus the small
// utility kernels (fill, streaming copy, strided gather) and the tuning table.
#include "hk_common.h"

#include <atomic>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

namespace hk {

static thread_local char g_last_error[512] = "";

void set_last_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int launch_check(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_last_error("launch of %s failed: %s", what, hipGetErrorString(e));
    return HK_ERR_HIP;
  }
  return HK_OK;
}

static thread_local hipEvent_t g_prof_before = nullptr;   // armed by hk_profile_next_kernel()
static thread_local hipEvent_t g_prof_after = nullptr;
static thread_local hipEvent_t g_pend_before = nullptr;   // handed to the next HK_LAUNCH by profile_before()
static thread_local hipEvent_t g_pend_after = nullptr;

void profile_before(hipStream_t) {
  g_pend_before = g_prof_before;
  g_pend_after = g_prof_after;
  g_prof_before = g_prof_after = nullptr;
}
void profile_after(hipStream_t) {
  g_pend_before = g_pend_after = nullptr;
}
bool profile_claim(hipEvent_t* before, hipEvent_t* after) {
  if (!g_pend_before || !g_pend_after) return false;
  *before = g_pend_before;
  *after = g_pend_after;
  g_pend_before = g_pend_after = nullptr;
  return true;
}

// ---------------------------------------------------------------------------
// tuning table
// ---------------------------------------------------------------------------
static const char* const kTuneNames[] = {
  "norm_fwd_threads",   // threads cooperating on one row (64 = one wavefront per row)
  "norm_bwd_threads",
  "norm_bwd_blocks",    // persistent grid size of the backward kernels
  "softmax_threads",
  "sce_threads",
  "reduce_inner_threads",
  "reduce_outer_row_blocks",
  "norm_bwd_rows_per_block",
  "norm_bwd_prefetch",  // rows loaded ahead by the backward kernel (1..3)
  "reduce_outer_waves_across",  // wavefronts of a column-reduction workgroup side by side across columns
  "reduce_outer_waves",         // wavefronts of a column-reduction workgroup in all
  "norm_fwd_rows",              // rows a workgroup of the forward norm kernel takes (1 or 2)
  "norm_fwd_resident",         // workgroups of the two-row forward norm kernel resident per compute unit (-1: no cap)
};
constexpr int kNumTune = sizeof(kTuneNames) / sizeof(kTuneNames[0]);
static_assert(kNumTune == TUNE_NUM_KEYS, "tune name table out of sync with TuneKey");
// process-wide; written by hk_tune_set from any thread, read by every launch plan: relaxed atomics
static std::atomic<int> g_tune[kNumTune];

int tune_get(int key) { return (key >= 0 && key < kNumTune) ? g_tune[key].load(std::memory_order_relaxed) : 0; }

// Compute-unit count of the current device, cached per device index.
int device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// LDS of the current device, cached per device index: bytes one compute unit holds and bytes one workgroup may ask
// for.  What the device reports is used; the figures of this part (160 KB, 64 KB) only stand in when the query fails.
void device_lds_bytes(size_t* per_cu, size_t* per_block) {
  static size_t cached_cu[64] = {0}, cached_block[64] = {0};
  int dev = 0;
  size_t cu = 160 * 1024, block = 64 * 1024;
  if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
    if (cached_cu[dev] == 0) {
      int a = 0, b = 0;
      if (hipDeviceGetAttribute(&a, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || a <= 0)
        a = int(cu);
      if (hipDeviceGetAttribute(&b, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || b <= 0)
        b = int(block);
      cached_cu[dev] = size_t(a);
      cached_block[dev] = size_t(b);
    }
    cu = cached_cu[dev];
    block = cached_block[dev];
  }
  *per_cu = cu;
  *per_block = block;
}

// ---------------------------------------------------------------------------
// utility kernels
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fill_bytes_kernel(uint8_t* dst, uint32_t word, size_t bytes) {
  // head / tail bytes individually (first workgroup), the aligned middle as 16-byte stores: every
  // thread writes one vector and retires, the shape that streams fastest here (more stores per thread
  // measured 10 % slower)
  constexpr int UNROLL = 1;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
  size_t head = (16 - (addr & 15)) & 15;
  if (head > bytes) head = bytes;
  const size_t nvec = (bytes - head) / 16;
  const size_t tail_begin = head + nvec * 16;
  const uint8_t b = uint8_t(word & 0xff);
  if (blockIdx.x == 0) {
    if (threadIdx.x < head) dst[threadIdx.x] = b;
    if (threadIdx.x < bytes - tail_begin) dst[tail_begin + threadIdx.x] = b;
  }
  const u32x4 v = {word, word, word, word};
  u32x4* mid = reinterpret_cast<u32x4*>(dst + head);
  const size_t base = (size_t(blockIdx.x) * UNROLL) * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < UNROLL; ++i) {
    const size_t idx = base + size_t(i) * 256;
    if (idx < nvec) mid[idx] = v;
  }
}

// the copy in the shape that streams fastest: one-wavefront workgroups, non-temporal loads and stores
template <int UNROLL>
__global__ __launch_bounds__(kStreamThreads) void copy16_kernel(u32x4* __restrict__ dst,
                                                                const u32x4* __restrict__ src, size_t nvec) {
  const size_t base = (size_t(blockIdx.x) * UNROLL) * kStreamThreads + threadIdx.x;
  u32x4 v[UNROLL];
#pragma unroll
  for (int i = 0; i < UNROLL; ++i) {
    size_t idx = base + size_t(i) * kStreamThreads;
    if (idx < nvec) v[i] = ld16(src + idx);
  }
#pragma unroll
  for (int i = 0; i < UNROLL; ++i) {
    size_t idx = base + size_t(i) * kStreamThreads;
    if (idx < nvec) st16_stream(dst + idx, v[i]);
  }
}

struct StridedMeta {
  int ndim;
  int64_t shape[8];
  int64_t stride[8];
};

// SCATTER = false: dst (dense) <- src laid out by m; SCATTER = true: dst laid out by m <- src (dense)
template <typename W, bool SCATTER>
__global__ __launch_bounds__(256) void strided_copy_kernel(const W* __restrict__ src,
                                                           W* __restrict__ dst, StridedMeta m,
                                                           int64_t numel) {
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (; i < numel; i += step) {
    int64_t rem = i, off = 0;
    for (int d = m.ndim - 1; d >= 0; --d) {
      int64_t q = rem / m.shape[d];
      off += (rem - q * m.shape[d]) * m.stride[d];
      rem = q;
    }
    if constexpr (SCATTER) dst[off] = src[i];
    else dst[i] = src[off];
  }
}

// Rows that are contiguous on both sides, as 16-byte vectors: one vector per thread, one-wavefront workgroups,
// non-temporal loads and stores (the shape that streams a read + write mix fastest).  m counts in vectors.
template <bool SCATTER>
__global__ __launch_bounds__(kStreamThreads) void strided_rows_vec_kernel(const u32x4* __restrict__ src,
                                                                          u32x4* __restrict__ dst, StridedMeta m,
                                                                          int64_t nvec) {
  const int64_t i = int64_t(blockIdx.x) * kStreamThreads + threadIdx.x;
  if (i >= nvec) return;
  int64_t rem = i, off = 0;
  for (int d = m.ndim - 1; d >= 0; --d) {
    const int64_t q = rem / m.shape[d];
    off += (rem - q * m.shape[d]) * m.stride[d];
    rem = q;
  }
  if constexpr (SCATTER) st16_stream(dst + off, ld16(src + i));
  else st16_stream(dst + i, ld16(src + off));
}

// The same copy for a view whose unit-stride dimension is not the last one (a transposed or permuted array):
// 64 x 64 tiles of the two dimensions that are contiguous on one side each go through LDS, so that both the reads
// and the writes of a wavefront are consecutive in memory.  u = the view's unit-stride dimension, v = the last
// dimension (unit stride in the dense array); the other dimensions are walked by the workgroup index.
struct TransposeMeta {
  int n_other;
  int64_t other_shape[6], other_dense[6], other_view[6];
  int64_t U, V;        // extents of u and v
  int64_t u_dense;     // stride of u in the dense array
  int64_t v_view;      // stride of v in the view
  int64_t tiles_u, tiles_v;
};

template <typename W, bool SCATTER>
__global__ __launch_bounds__(256) void strided_transpose_kernel(const W* __restrict__ src, W* __restrict__ dst,
                                                                TransposeMeta m) {
  constexpr int TS = 64;
  __shared__ W tile[TS][TS + 1];
  int64_t b = blockIdx.x;
  const int64_t tv = b % m.tiles_v;
  b /= m.tiles_v;
  const int64_t tu = b % m.tiles_u;
  b /= m.tiles_u;
  int64_t base_dense = 0, base_view = 0;
  for (int d = m.n_other - 1; d >= 0; --d) {
    const int64_t q = b / m.other_shape[d], idx = b - q * m.other_shape[d];
    base_dense += idx * m.other_dense[d];
    base_view += idx * m.other_view[d];
    b = q;
  }
  const int tx = int(threadIdx.x & 63), ty = int(threadIdx.x >> 6);
  const int64_t u0 = tu * TS, v0 = tv * TS;
  const W* dense_in = src + base_dense;
  const W* view_in = src + base_view;
  W* dense_out = dst + base_dense;
  W* view_out = dst + base_view;
  if constexpr (!SCATTER) {
    for (int j = ty; j < TS; j += 4) {             // lanes run along u: consecutive in the view
      const int64_t u = u0 + tx, v = v0 + j;
      if (u < m.U && v < m.V) tile[j][tx] = view_in[u + v * m.v_view];
    }
    __syncthreads();
    for (int j = ty; j < TS; j += 4) {             // lanes run along v: consecutive in the dense array
      const int64_t u = u0 + j, v = v0 + tx;
      if (u < m.U && v < m.V) dense_out[u * m.u_dense + v] = tile[tx][j];
    }
  } else {
    for (int j = ty; j < TS; j += 4) {
      const int64_t u = u0 + j, v = v0 + tx;
      if (u < m.U && v < m.V) tile[j][tx] = dense_in[u * m.u_dense + v];
    }
    __syncthreads();
    for (int j = ty; j < TS; j += 4) {
      const int64_t u = u0 + tx, v = v0 + j;
      if (u < m.U && v < m.V) view_out[u + v * m.v_view] = tile[tx][j];
    }
  }
}

// The same tiles moved as 16-byte vectors on both sides (K = 16 / sizeof(W) elements each): a lane reads K
// consecutive elements of the side it is reading and writes K consecutive elements of the other side, the exchange
// happening in LDS.  Needs every extent, stride and address involved to be a multiple of K elements.
template <typename W, bool SCATTER>
__global__ __launch_bounds__(256) void strided_transpose_vec_kernel(const W* __restrict__ src, W* __restrict__ dst,
                                                                    TransposeMeta m) {
  constexpr int TS = 64, K = 16 / int(sizeof(W));
  constexpr int LPR = TS / K;          // lanes along a tile row
  constexpr int RPP = 256 / LPR;       // tile rows per pass of the workgroup
  constexpr int PAD = sizeof(W) >= 4 ? 1 : 2;   // keeps the column reads below off each other's banks
  __shared__ W tile[TS][TS + PAD];
  int64_t b = blockIdx.x;
  const int64_t tv = b % m.tiles_v;
  b /= m.tiles_v;
  // diagonal order: workgroups that run together differ in both tile coordinates, so their rows do not all sit the
  // same power-of-two pitch apart (a transposed fp32 [8192 x 4096]: 56.9 -> 49.6 us)
  const int64_t tu = (b % m.tiles_u + tv) % m.tiles_u;
  b /= m.tiles_u;
  int64_t base_dense = 0, base_view = 0;
  for (int d = m.n_other - 1; d >= 0; --d) {
    const int64_t q = b / m.other_shape[d], idx = b - q * m.other_shape[d];
    base_dense += idx * m.other_dense[d];
    base_view += idx * m.other_view[d];
    b = q;
  }
  const int cl = int(threadIdx.x) % LPR, rl = int(threadIdx.x) / LPR;
  const int64_t u0 = tu * TS, v0 = tv * TS;
  union Vec { u32x4 raw; W e[K]; };
  if constexpr (!SCATTER) {
    const W* view_in = src + base_view;
    W* dense_out = dst + base_dense;
    for (int j = rl; j < TS; j += RPP) {           // tile[v][u], vectors along u
      const int64_t u = u0 + cl * K, v = v0 + j;
      if (u < m.U && v < m.V) {
        Vec x;
        x.raw = ld16(view_in + u + v * m.v_view);
#pragma unroll
        for (int k = 0; k < K; ++k) tile[j][cl * K + k] = x.e[k];
      }
    }
    __syncthreads();
    for (int i = rl; i < TS; i += RPP) {           // vectors along v
      const int64_t u = u0 + i, v = v0 + cl * K;
      if (u < m.U && v < m.V) {
        Vec x;
#pragma unroll
        for (int k = 0; k < K; ++k) x.e[k] = tile[cl * K + k][i];
        st16_stream(dense_out + u * m.u_dense + v, x.raw);
      }
    }
  } else {
    const W* dense_in = src + base_dense;
    W* view_out = dst + base_view;
    for (int j = rl; j < TS; j += RPP) {           // tile[u][v], vectors along v
      const int64_t u = u0 + j, v = v0 + cl * K;
      if (u < m.U && v < m.V) {
        Vec x;
        x.raw = ld16(dense_in + u * m.u_dense + v);
#pragma unroll
        for (int k = 0; k < K; ++k) tile[j][cl * K + k] = x.e[k];
      }
    }
    __syncthreads();
    for (int i = rl; i < TS; i += RPP) {           // vectors along u
      const int64_t u = u0 + cl * K, v = v0 + i;
      if (u < m.U && v < m.V) {
        Vec x;
#pragma unroll
        for (int k = 0; k < K; ++k) x.e[k] = tile[cl * K + k][i];
        st16_stream(view_out + u + v * m.v_view, x.raw);
      }
    }
  }
}

} // namespace hk

using namespace hk;

template <bool SCATTER>
static int strided_copy_any(const char* who, int dtype, const void* src, void* dst, int ndim, const int64_t* shape,
                            const int64_t* strides, hkStream_t stream) {
  HK_REQUIRE(ndim >= 0 && ndim <= 8, HK_ERR_INVALID, "%s: ndim %d not in [0, 8]", who, ndim);
  HK_REQUIRE(ndim == 0 || (shape && strides), HK_ERR_INVALID, "%s: null meta", who);
  size_t es = dtype_size(dtype);
  HK_REQUIRE(es != 0, HK_ERR_UNSUPPORTED, "%s: unknown dtype %d", who, dtype);
  // extents of 1 carry no index; neighbours that the view steps through like one dimension become one
  StridedMeta m;
  m.ndim = 0;
  int64_t numel = 1;
  for (int d = 0; d < ndim; ++d) {
    HK_REQUIRE(shape[d] >= 0, HK_ERR_INVALID, "%s: negative extent", who);
    numel *= shape[d];
    if (shape[d] == 1) continue;
    if (m.ndim > 0 && m.stride[m.ndim - 1] == strides[d] * shape[d]) {
      m.shape[m.ndim - 1] *= shape[d];
      m.stride[m.ndim - 1] = strides[d];
    } else {
      m.shape[m.ndim] = shape[d];
      m.stride[m.ndim] = strides[d];
      ++m.ndim;
    }
  }
  if (numel == 0) return HK_OK;
  HK_REQUIRE(src && dst, HK_ERR_INVALID, "%s: null pointer", who);
  hipStream_t s = as_hip(stream);
  profile_before(s);

  // a permuted view: the dimension it is contiguous in is not the last one
  const int v = m.ndim - 1;
  int u = -1;
  if (m.ndim >= 2 && m.stride[v] != 1 && m.shape[v] >= 16) {
    for (int d = 0; d < v; ++d)
      if (m.stride[d] == 1 && m.shape[d] >= 16 && (u < 0 || m.shape[d] > m.shape[u])) u = d;
  }
  if (u >= 0) {
    TransposeMeta t;
    t.n_other = 0;
    int64_t dense_stride = 1, others = 1;
    int64_t dense_of[8];
    for (int d = m.ndim - 1; d >= 0; --d) { dense_of[d] = dense_stride; dense_stride *= m.shape[d]; }
    t.u_dense = dense_of[u];
    for (int d = 0; d < m.ndim; ++d) {
      if (d == u || d == v) continue;
      t.other_shape[t.n_other] = m.shape[d];
      t.other_dense[t.n_other] = dense_of[d];
      t.other_view[t.n_other] = m.stride[d];
      ++t.n_other;
      others *= m.shape[d];
    }
    t.U = m.shape[u];
    t.V = m.shape[v];
    t.v_view = m.stride[v];
    t.tiles_u = (t.U + 63) / 64;
    t.tiles_v = (t.V + 63) / 64;
    const int64_t nblocks = t.tiles_u * t.tiles_v * others;
    // whole 16-byte vectors on both sides?
    const int64_t k = es >= 2 ? int64_t(16 / es) : 0;
    bool vec = k > 0 && t.U % k == 0 && t.V % k == 0 && t.v_view % k == 0 &&
               reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
    for (int d = 0; d < t.n_other && vec; ++d) vec = t.other_view[d] % k == 0;
    if (nblocks <= 0x7fffffffLL && vec) {
      dim3 g{unsigned(nblocks)}, b{256};
      switch (es) {
        case 2: HK_LAUNCH((strided_transpose_vec_kernel<uint16_t, SCATTER>), g, b, 0, s, (const uint16_t*)src, (uint16_t*)dst, t); break;
        case 4: HK_LAUNCH((strided_transpose_vec_kernel<uint32_t, SCATTER>), g, b, 0, s, (const uint32_t*)src, (uint32_t*)dst, t); break;
        default: HK_LAUNCH((strided_transpose_vec_kernel<uint64_t, SCATTER>), g, b, 0, s, (const uint64_t*)src, (uint64_t*)dst, t); break;
      }
      profile_after(s);
      return launch_check("strided_transpose_vec_kernel");
    }
    if (nblocks <= 0x7fffffffLL) {
      dim3 g{unsigned(nblocks)}, b{256};
      switch (es) {
        case 1: HK_LAUNCH((strided_transpose_kernel<uint8_t, SCATTER>), g, b, 0, s, (const uint8_t*)src, (uint8_t*)dst, t); break;
        case 2: HK_LAUNCH((strided_transpose_kernel<uint16_t, SCATTER>), g, b, 0, s, (const uint16_t*)src, (uint16_t*)dst, t); break;
        case 4: HK_LAUNCH((strided_transpose_kernel<uint32_t, SCATTER>), g, b, 0, s, (const uint32_t*)src, (uint32_t*)dst, t); break;
        default: HK_LAUNCH((strided_transpose_kernel<uint64_t, SCATTER>), g, b, 0, s, (const uint64_t*)src, (uint64_t*)dst, t); break;
      }
      profile_after(s);
      return launch_check("strided_transpose_kernel");
    }
  }

  // rows that are contiguous on both sides and made of whole 16-byte vectors move as vectors
  if (m.ndim >= 1 && m.stride[v] == 1 && es < 16) {
    const int64_t k = int64_t(16 / es);
    bool ok = m.shape[v] % k == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(dst) % 16 == 0;
    for (int d = 0; d < v; ++d) ok = ok && m.stride[d] % k == 0;
    if (ok) {
      m.shape[v] /= k;
      for (int d = 0; d < v; ++d) m.stride[d] /= k;
      numel /= k;
      es = 16;
      const int64_t nb = (numel + kStreamThreads - 1) / kStreamThreads;
      if (nb <= 0x7fffffffLL) {
        HK_LAUNCH((strided_rows_vec_kernel<SCATTER>), dim3{unsigned(nb)}, dim3{unsigned(kStreamThreads)}, 0, s,
                  (const u32x4*)src, (u32x4*)dst, m, numel);
        profile_after(s);
        return launch_check("strided_rows_vec_kernel");
      }
    }
  }
  int64_t blocks = (numel + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  dim3 g{unsigned(blocks)}, b{256};
  switch (es) {
    case 16: HK_LAUNCH((strided_copy_kernel<u32x4, SCATTER>), g, b, 0, s, (const u32x4*)src, (u32x4*)dst, m, numel); break;
    case 1: HK_LAUNCH((strided_copy_kernel<uint8_t, SCATTER>), g, b, 0, s, (const uint8_t*)src, (uint8_t*)dst, m, numel); break;
    case 2: HK_LAUNCH((strided_copy_kernel<uint16_t, SCATTER>), g, b, 0, s, (const uint16_t*)src, (uint16_t*)dst, m, numel); break;
    case 4: HK_LAUNCH((strided_copy_kernel<uint32_t, SCATTER>), g, b, 0, s, (const uint32_t*)src, (uint32_t*)dst, m, numel); break;
    default: HK_LAUNCH((strided_copy_kernel<uint64_t, SCATTER>), g, b, 0, s, (const uint64_t*)src, (uint64_t*)dst, m, numel); break;
  }
  profile_after(s);
  return launch_check("strided_copy_kernel");
}

extern "C" {

const char* hk_last_error(void) { return g_last_error; }
const char* hk_version(void) { return "hk_rowwise 0.1 (gfx950)"; }

int hk_device_count(int* count) {
  HK_REQUIRE(count, HK_ERR_INVALID, "hk_device_count: null output");
  HK_CHECK_HIP(hipGetDeviceCount(count));
  return HK_OK;
}
int hk_set_device(int device) { HK_CHECK_HIP(hipSetDevice(device)); return HK_OK; }
int hk_get_device(int* device) {
  HK_REQUIRE(device, HK_ERR_INVALID, "hk_get_device: null output");
  HK_CHECK_HIP(hipGetDevice(device));
  return HK_OK;
}
int hk_device_sync(void) { HK_CHECK_HIP(hipDeviceSynchronize()); return HK_OK; }
int hk_mem_get_info(size_t* free_bytes, size_t* total_bytes) {
  HK_REQUIRE(free_bytes && total_bytes, HK_ERR_INVALID, "hk_mem_get_info: null output");
  HK_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return HK_OK;
}
int hk_device_cu_count(int device, int* cus) {
  HK_REQUIRE(cus, HK_ERR_INVALID, "hk_device_cu_count: null output");
  HK_CHECK_HIP(hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, device));
  return HK_OK;
}

int hk_device_lds_bytes(int device, size_t* per_cu, size_t* per_block) {
  HK_REQUIRE(per_cu && per_block, HK_ERR_INVALID, "hk_device_lds_bytes: null output");
  int a = 0, b = 0;
  HK_CHECK_HIP(hipDeviceGetAttribute(&a, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device));
  HK_CHECK_HIP(hipDeviceGetAttribute(&b, hipDeviceAttributeMaxSharedMemoryPerBlock, device));
  *per_cu = size_t(a);
  *per_block = size_t(b);
  return HK_OK;
}

int hk_malloc(void** ptr, size_t bytes) {
  HK_REQUIRE(ptr, HK_ERR_INVALID, "hk_malloc: null output");
  *ptr = nullptr;
  if (bytes == 0) return HK_OK;
  const hipError_t e = hipMalloc(ptr, bytes);
  if (e != hipSuccess) {
    // the runtime keeps a failed call as its "last error": take it out, or the launch check of the next
    // kernel (after a caller has freed memory and retried) would report this failure as its own
    (void)hipGetLastError();
    *ptr = nullptr;
    set_last_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return HK_ERR_HIP;
  }
  return HK_OK;
}
int hk_free(void* ptr) {
  if (ptr) HK_CHECK_HIP(hipFree(ptr));
  return HK_OK;
}
int hk_host_malloc(void** ptr, size_t bytes) {
  HK_REQUIRE(ptr, HK_ERR_INVALID, "hk_host_malloc: null output");
  *ptr = nullptr;
  if (bytes == 0) return HK_OK;
  const hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *ptr = nullptr;
    set_last_error("hipHostMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return HK_ERR_HIP;
  }
  return HK_OK;
}
int hk_host_free(void* ptr) {
  if (ptr) HK_CHECK_HIP(hipHostFree(ptr));
  return HK_OK;
}
int hk_memcpy_h2d(void* dst, const void* src, size_t bytes, hkStream_t stream) {
  if (bytes == 0) return HK_OK;
  HK_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_hip(stream)));
  return HK_OK;
}
int hk_memcpy_d2h(void* dst, const void* src, size_t bytes, hkStream_t stream) {
  if (bytes == 0) return HK_OK;
  HK_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_hip(stream)));
  return HK_OK;
}
int hk_memcpy_d2d(void* dst, const void* src, size_t bytes, hkStream_t stream) {
  if (bytes == 0) return HK_OK;
  HK_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_hip(stream)));
  return HK_OK;
}
int hk_memset(void* dst, int value, size_t bytes, hkStream_t stream) {
  if (bytes == 0) return HK_OK;
  HK_REQUIRE(dst, HK_ERR_INVALID, "hk_memset: null destination");
  uint32_t b = uint32_t(value) & 0xff;
  uint32_t word = b | (b << 8) | (b << 16) | (b << 24);
  size_t nvec = bytes / 16 + 1;
  size_t blocks = (nvec + 255) / 256;
  HK_REQUIRE(blocks <= 0x7fffffffu, HK_ERR_INVALID, "hk_memset: size too large");
  profile_before(as_hip(stream));
  HK_LAUNCH(fill_bytes_kernel, dim3(unsigned(blocks)), dim3(256), 0, as_hip(stream),
                     static_cast<uint8_t*>(dst), word, bytes);
  profile_after(as_hip(stream));
  return launch_check("fill_bytes_kernel");
}

int hk_stream_create(hkStream_t* stream) {
  HK_REQUIRE(stream, HK_ERR_INVALID, "hk_stream_create: null output");
  hipStream_t s;
  HK_CHECK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = reinterpret_cast<hkStream_t>(s);
  return HK_OK;
}
int hk_stream_destroy(hkStream_t stream) {
  if (stream) HK_CHECK_HIP(hipStreamDestroy(as_hip(stream)));
  return HK_OK;
}
int hk_stream_sync(hkStream_t stream) {
  HK_CHECK_HIP(hipStreamSynchronize(as_hip(stream)));
  return HK_OK;
}
int hk_stream_wait_event(hkStream_t stream, hkEvent_t event) {
  HK_REQUIRE(event, HK_ERR_INVALID, "hk_stream_wait_event: null event");
  HK_CHECK_HIP(hipStreamWaitEvent(as_hip(stream), reinterpret_cast<hipEvent_t>(event), 0));
  return HK_OK;
}

int hk_event_create(hkEvent_t* event, int enable_timing) {
  HK_REQUIRE(event, HK_ERR_INVALID, "hk_event_create: null output");
  hipEvent_t e;
  HK_CHECK_HIP(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming));
  *event = reinterpret_cast<hkEvent_t>(e);
  return HK_OK;
}
int hk_event_destroy(hkEvent_t event) {
  if (event) HK_CHECK_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return HK_OK;
}
int hk_event_record(hkEvent_t event, hkStream_t stream) {
  HK_REQUIRE(event, HK_ERR_INVALID, "hk_event_record: null event");
  HK_CHECK_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_hip(stream)));
  return HK_OK;
}
int hk_event_sync(hkEvent_t event) {
  HK_REQUIRE(event, HK_ERR_INVALID, "hk_event_sync: null event");
  HK_CHECK_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
  return HK_OK;
}
int hk_event_query(hkEvent_t event, int* done) {
  HK_REQUIRE(event && done, HK_ERR_INVALID, "hk_event_query: null argument");
  hipError_t e = hipEventQuery(reinterpret_cast<hipEvent_t>(event));
  if (e == hipSuccess) { *done = 1; return HK_OK; }
  if (e == hipErrorNotReady) { *done = 0; (void)hipGetLastError(); return HK_OK; }
  set_last_error("hipEventQuery failed: %s", hipGetErrorString(e));
  return HK_ERR_HIP;
}
int hk_event_elapsed_ns(hkEvent_t start, hkEvent_t stop, int64_t* ns) {
  HK_REQUIRE(start && stop && ns, HK_ERR_INVALID, "hk_event_elapsed_ns: null argument");
  float ms = 0.f;
  HK_CHECK_HIP(hipEventElapsedTime(&ms, reinterpret_cast<hipEvent_t>(start),
                                   reinterpret_cast<hipEvent_t>(stop)));
  *ns = int64_t(double(ms) * 1.0e6);
  return HK_OK;
}

int hk_profile_next_kernel(hkEvent_t before, hkEvent_t after) {
  g_prof_before = reinterpret_cast<hipEvent_t>(before);
  g_prof_after = reinterpret_cast<hipEvent_t>(after);
  return HK_OK;
}

int hk_tune_set(const char* key, int value) {
  HK_REQUIRE(key, HK_ERR_INVALID, "hk_tune_set: null key");
  for (int i = 0; i < kNumTune; ++i) {
    if (std::strcmp(key, kTuneNames[i]) == 0) {
      g_tune[i].store(value, std::memory_order_relaxed);
      return HK_OK;
    }
  }
  set_last_error("hk_tune_set: unknown key '%s'", key);
  return HK_ERR_INVALID;
}

const char* hk_tune_keys(void) {
  static std::string keys;
  static std::once_flag once;
  std::call_once(once, [] {
    for (int i = 0; i < kNumTune; ++i) {
      if (i) keys += ",";
      keys += kTuneNames[i];
    }
  });
  return keys.c_str();
}

int hk_copy_kernel(void* dst, const void* src, size_t bytes, hkStream_t stream) {
  if (bytes == 0) return HK_OK;
  HK_REQUIRE(dst && src, HK_ERR_INVALID, "hk_copy_kernel: null pointer");
  HK_REQUIRE(bytes % 16 == 0 && aligned16(dst) && aligned16(src), HK_ERR_INVALID,
             "hk_copy_kernel: needs 16-byte aligned pointers and size");
  constexpr int UNROLL = 1;
  size_t nvec = bytes / 16;
  size_t blocks = (nvec + kStreamThreads * UNROLL - 1) / (kStreamThreads * UNROLL);
  HK_REQUIRE(blocks <= 0x7fffffffu, HK_ERR_INVALID, "hk_copy_kernel: size too large");
  profile_before(as_hip(stream));
  HK_LAUNCH(copy16_kernel<UNROLL>, dim3(unsigned(blocks)), dim3(kStreamThreads), 0, as_hip(stream),
                     static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), nvec);
  profile_after(as_hip(stream));
  return launch_check("copy16_kernel");
}

int hk_strided_copy(int dtype, const void* src, void* dst, int ndim, const int64_t* shape,
                    const int64_t* src_strides, hkStream_t stream) {
  return strided_copy_any<false>("hk_strided_copy", dtype, src, dst, ndim, shape, src_strides, stream);
}

int hk_strided_scatter(int dtype, const void* src, void* dst, int ndim, const int64_t* shape,
                       const int64_t* dst_strides, hkStream_t stream) {
  return strided_copy_any<true>("hk_strided_scatter", dtype, src, dst, ndim, shape, dst_strides, stream);
}

} // extern "C"
