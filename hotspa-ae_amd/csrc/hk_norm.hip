// LayerNorm / RMSNorm forward and backward for gfx950: dtype dispatch and the C entry points.  The kernels are
// in hk_norm_fwd_impl.h / hk_norm_bwd_impl.h, instantiated per storage type in hk_norm_{fwd,bwd}_*.hip.
#include "hk_norm.h"

#include <mutex>

namespace hk {

static int norm_fwd_dispatch(int dtype, NormFwdArgs& a, hipStream_t s, const char* who) {
  HK_REQUIRE(a.rows >= 0 && a.cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  if (a.rows == 0 || a.cols == 0) return HK_OK;
  HK_REQUIRE(a.rows <= 0x7fffffffLL && a.cols <= 0x3fffffff, HK_ERR_INVALID,
             "%s: shape [%lld, %d] too large", who, (long long)a.rows, a.cols);
  HK_REQUIRE(a.x && a.y, HK_ERR_INVALID, "%s: null input/output", who);
  if (a.n0 == 0) { a.n0 = a.rows; a.n1 = a.n2 = 1; a.rn = RowNumbering{1, 0, 0}; }   // one level
  HK_REQUIRE(a.n0 == 1 || (a.x_pitch >= a.cols && a.y_pitch >= a.cols && (!a.residual || a.res_pitch >= a.cols) &&
                           (!a.x_out || a.xout_pitch >= a.cols)), HK_ERR_INVALID,
             "%s: a row pitch is smaller than the %d columns of a row", who, a.cols);
  a.inv_cols = 1.0f / float(a.cols);
  switch (dtype) {
    case HK_FLOAT32: return norm_fwd_typed<float>(a, s);
    case HK_BFLOAT16: return norm_fwd_typed<bf16>(a, s);
    case HK_FLOAT16: return norm_fwd_typed<fp16>(a, s);
    case HK_FLOAT64: return norm_fwd_f64(a, s);
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

static int norm_bwd_dispatch(int dtype, NormBwdArgs& a, int mode, void* dgamma, void* dbeta,
                             void* ws, size_t ws_bytes, hipStream_t s, const char* who) {
  HK_REQUIRE(a.rows >= 0 && a.cols >= 0, HK_ERR_INVALID, "%s: negative shape", who);
  if (a.rows == 0 || a.cols == 0) return HK_OK;
  HK_REQUIRE(a.rows <= 0x7fffffffLL && a.cols <= 0x3fffffff, HK_ERR_INVALID,
             "%s: shape [%lld, %d] too large", who, (long long)a.rows, a.cols);
  HK_REQUIRE(a.dy && a.x && a.dx && a.stat, HK_ERR_INVALID, "%s: null input/output", who);
  HK_REQUIRE(mode != BWD_LN || a.mean, HK_ERR_INVALID, "%s: mean is required", who);
  if (a.n0 == 0) { a.n0 = a.rows; a.n1 = a.n2 = 1; a.rn = RowNumbering{1, 0, 0}; }   // one level
  HK_REQUIRE(a.n0 == 1 || (a.dy_pitch >= a.cols && a.x_pitch >= a.cols && a.dx_pitch >= a.cols &&
                           (!a.dx_in || a.dxin_pitch >= a.cols) && (!a.dres || a.dres_pitch >= a.cols)), HK_ERR_INVALID,
             "%s: a row pitch is smaller than the %d columns of a row", who, a.cols);
  a.inv_cols = 1.0f / float(a.cols);
  switch (dtype) {
    case HK_FLOAT32: return norm_bwd_typed<float>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_BFLOAT16: return norm_bwd_typed<bf16>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_FLOAT16: return norm_bwd_typed<fp16>(a, mode, dgamma, dbeta, ws, ws_bytes, s);
    case HK_FLOAT64: return norm_bwd_f64(a, mode, dgamma, dbeta, s);
    default:
      set_last_error("%s: not implemented for dtype %d", who, dtype);
      return HK_ERR_UNSUPPORTED;
  }
}

// level_rows = {n0, n1, n2} of a *_strided_rows call: no count negative, the product within the row limit.
// Writes the total.
static int check_levels(const int64_t level_rows[3], int64_t* rows, const char* who) {
  HK_REQUIRE(level_rows, HK_ERR_INVALID, "%s: null level_rows", who);
  const int64_t n0 = level_rows[0], n1 = level_rows[1], n2 = level_rows[2];
  HK_REQUIRE(n0 >= 0 && n1 >= 0 && n2 >= 0, HK_ERR_INVALID, "%s: negative level count", who);
  if (n0 == 0 || n1 == 0 || n2 == 0) { *rows = 0; return HK_OK; }
  HK_REQUIRE(n0 <= 0x7fffffffLL && n0 * n1 <= 0x7fffffffLL && n0 * n1 * n2 <= 0x7fffffffLL, HK_ERR_INVALID,
             "%s: too many rows", who);
  *rows = n0 * n1 * n2;
  return HK_OK;
}

// per level, the sum of the steps of the operands that are there: what the walk order is chosen by
static void add_steps(int64_t key[3], const void* operand, const int64_t steps[3]) {
  if (operand == nullptr || steps == nullptr) return;
  for (int k = 0; k < 3; ++k) key[k] += steps[k];
}

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


int hk_layer_norm_fwd_strided_rows(int dtype, const void* x, const int64_t x_steps[3], const void* gamma,
                                   const void* beta, void* y, const int64_t y_steps[3], void* mean, void* stat,
                                   int stats_dtype, int stat_kind, const int64_t level_rows[3], int64_t cols,
                                   float eps, hkStream_t stream) {
  const char* who = "hk_layer_norm_fwd_strided_rows";
  HK_REQUIRE(x_steps && y_steps, HK_ERR_INVALID, "%s: null steps", who);
  int64_t rows = 0;
  int rc = check_levels(level_rows, &rows, who);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(stats_dtype == HK_FLOAT32 || stats_dtype == dtype, HK_ERR_INVALID,
             "%s: stats dtype %d must be fp32 or the data dtype %d", who, stats_dtype, dtype);
  HK_REQUIRE(stat_kind == HK_STAT_VAR || stat_kind == HK_STAT_RSTD, HK_ERR_INVALID, "%s: bad stat_kind %d", who,
             stat_kind);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  HK_REQUIRE(dtype != HK_FLOAT64 || stats_dtype == HK_FLOAT64, HK_ERR_UNSUPPORTED,
             "%s: fp64 data needs fp64 statistics", who);
  NormFwdArgs a{};
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y; a.mean = mean; a.stat = stat;
  int64_t key[3] = {0, 0, 0};
  add_steps(key, x, x_steps);
  add_steps(key, y, y_steps);
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  walk_steps(w, x_steps, &a.x_pitch, &a.x_lv);
  walk_steps(w, y_steps, &a.y_pitch, &a.y_lv);
  a.n0 = w.n[0]; a.n1 = w.n[1]; a.n2 = w.n[2]; a.rn = w.rn;
  HK_REQUIRE(rows == 0 || walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)level_rows[0], (long long)level_rows[1], (long long)level_rows[2]);
  a.rows = rows; a.cols = int(cols); a.eps = eps; a.is_rms = 0; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  return norm_fwd_dispatch(dtype, a, as_hip(stream), who);
}

int hk_layer_norm_fwd_pitched(int dtype, const void* x, int64_t x_pitch, const void* gamma, const void* beta,
                              void* y, int64_t y_pitch, void* mean, void* stat, int stats_dtype, int stat_kind,
                              int64_t rows, int64_t cols, float eps, hkStream_t stream) {
  HK_REQUIRE(stats_dtype == HK_FLOAT32 || stats_dtype == dtype, HK_ERR_INVALID,
             "hk_layer_norm_fwd: stats dtype %d must be fp32 or the data dtype %d", stats_dtype, dtype);
  HK_REQUIRE(stat_kind == HK_STAT_VAR || stat_kind == HK_STAT_RSTD, HK_ERR_INVALID,
             "hk_layer_norm_fwd: bad stat_kind %d", stat_kind);
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_layer_norm_fwd: cols too large");
  NormFwdArgs a{};
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y; a.mean = mean; a.stat = stat;
  a.x_pitch = x_pitch; a.y_pitch = y_pitch;
  a.rows = rows; a.cols = int(cols); a.eps = eps; a.is_rms = 0; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  if (dtype == HK_FLOAT64) {
    HK_REQUIRE(stats_dtype == HK_FLOAT64, HK_ERR_UNSUPPORTED,
               "hk_layer_norm_fwd: fp64 data needs fp64 statistics");
  }
  return norm_fwd_dispatch(dtype, a, as_hip(stream), "hk_layer_norm_fwd");
}

int hk_layer_norm_fwd(int dtype, const void* x, const void* gamma, const void* beta, void* y,
                      void* mean, void* stat, int stats_dtype, int stat_kind, int64_t rows,
                      int64_t cols, float eps, hkStream_t stream) {
  return hk_layer_norm_fwd_pitched(dtype, x, cols, gamma, beta, y, cols, mean, stat, stats_dtype, stat_kind, rows,
                                   cols, eps, stream);
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

int hk_layer_norm_bwd_strided_rows(int dtype, const void* dy, const int64_t dy_steps[3], const void* x_or_y,
                                   const int64_t x_steps[3], const void* gamma, const void* beta, const void* mean,
                                   const void* stat, int stats_dtype, int stat_kind, void* dx,
                                   const int64_t dx_steps[3], void* dgamma, void* dbeta,
                                   const int64_t level_rows[3], int64_t cols, float eps, int memory_efficient,
                                   int clamp_gamma, void* workspace, size_t workspace_bytes, hkStream_t stream) {
  const char* who = "hk_layer_norm_bwd_strided_rows";
  HK_REQUIRE(dy_steps && x_steps && dx_steps, HK_ERR_INVALID, "%s: null steps", who);
  int64_t rows = 0;
  int rc = check_levels(level_rows, &rows, who);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(stats_dtype == HK_FLOAT32 || stats_dtype == dtype, HK_ERR_INVALID,
             "%s: stats dtype %d must be fp32 or the data dtype %d", who, stats_dtype, dtype);
  HK_REQUIRE(stat_kind == HK_STAT_VAR || stat_kind == HK_STAT_RSTD, HK_ERR_INVALID, "%s: bad stat_kind %d", who,
             stat_kind);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  HK_REQUIRE(dtype != HK_FLOAT64 || stats_dtype == HK_FLOAT64, HK_ERR_UNSUPPORTED,
             "%s: fp64 data needs fp64 statistics", who);
  NormBwdArgs a{};
  a.dy = dy; a.x = x_or_y; a.gamma = gamma; a.beta = beta; a.mean = mean; a.stat = stat;
  int64_t key[3] = {0, 0, 0};
  add_steps(key, dy, dy_steps);
  add_steps(key, x_or_y, x_steps);
  add_steps(key, dx, dx_steps);
  // the register kernel walks the rows itself; its fallback rides on a grid, whose limits the levels' own order meets
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  walk_steps(w, dy_steps, &a.dy_pitch, &a.dy_lv);
  walk_steps(w, x_steps, &a.x_pitch, &a.x_lv);
  walk_steps(w, dx_steps, &a.dx_pitch, &a.dx_lv);
  a.n0 = w.n[0]; a.n1 = w.n[1]; a.n2 = w.n[2]; a.rn = w.rn;
  HK_REQUIRE(rows == 0 || walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)level_rows[0], (long long)level_rows[1], (long long)level_rows[2]);
  a.dx = dx; a.rows = rows; a.cols = int(cols); a.eps = eps; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  a.clamp_gamma = clamp_gamma;
  return norm_bwd_dispatch(dtype, a, memory_efficient ? BWD_LN_MEMEFF : BWD_LN, dgamma, dbeta, workspace,
                           workspace_bytes, as_hip(stream), who);
}

int hk_layer_norm_bwd_pitched(int dtype, const void* dy, int64_t dy_pitch, const void* x_or_y, int64_t x_pitch,
                              const void* gamma, const void* beta, const void* mean, const void* stat,
                              int stats_dtype, int stat_kind, void* dx, int64_t dx_pitch, void* dgamma,
                              void* dbeta, int64_t rows, int64_t cols, float eps, int memory_efficient,
                              int clamp_gamma, void* workspace, size_t workspace_bytes, hkStream_t stream) {
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
  a.dy_pitch = dy_pitch; a.x_pitch = x_pitch; a.dx_pitch = dx_pitch;
  a.dx = dx; a.rows = rows; a.cols = int(cols); a.eps = eps; a.stat_kind = stat_kind;
  a.stats_f32 = (stats_dtype == HK_FLOAT32 && dtype != HK_FLOAT64) ? 1 : 0;
  a.clamp_gamma = clamp_gamma;
  return norm_bwd_dispatch(dtype, a, memory_efficient ? BWD_LN_MEMEFF : BWD_LN, dgamma, dbeta,
                           workspace, workspace_bytes, as_hip(stream), "hk_layer_norm_bwd");
}

int hk_layer_norm_bwd(int dtype, const void* dy, const void* x_or_y, const void* gamma,
                      const void* beta, const void* mean, const void* stat, int stats_dtype,
                      int stat_kind, void* dx, void* dgamma, void* dbeta, int64_t rows,
                      int64_t cols, float eps, int memory_efficient, int clamp_gamma,
                      void* workspace, size_t workspace_bytes, hkStream_t stream) {
  return hk_layer_norm_bwd_pitched(dtype, dy, cols, x_or_y, cols, gamma, beta, mean, stat, stats_dtype, stat_kind,
                                   dx, cols, dgamma, dbeta, rows, cols, eps, memory_efficient, clamp_gamma,
                                   workspace, workspace_bytes, stream);
}

static const int64_t kNoSteps[3] = {0, 0, 0};

int hk_dropout_add_ln_fwd_strided_rows(int itype, int rtype, int wtype, const void* x0, const int64_t x0_steps[3],
                                       const void* residual, const int64_t residual_steps[3], const void* gamma,
                                       const void* beta, void* z, const int64_t z_steps[3], void* x_out,
                                       const int64_t x_out_steps[3], void* mu, void* rsigma,
                                       const int64_t level_rows[3], int64_t cols, float eps, int is_rms_norm,
                                       hkStream_t stream) {
  const char* who = "hk_dropout_add_ln_fwd_strided_rows";
  HK_REQUIRE(x0_steps && z_steps && (!residual || residual_steps) && (!x_out || x_out_steps), HK_ERR_INVALID,
             "%s: null steps", who);
  if (!residual_steps) residual_steps = kNoSteps;
  if (!x_out_steps) x_out_steps = kNoSteps;
  int64_t rows = 0;
  int rc = check_levels(level_rows, &rows, who);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(itype == rtype && itype == wtype, HK_ERR_UNSUPPORTED,
             "%s: mixed dtypes (input %d, residual %d, weight %d) are not implemented", who, itype, rtype, wtype);
  HK_REQUIRE(itype == HK_FLOAT32 || itype == HK_BFLOAT16 || itype == HK_FLOAT16, HK_ERR_UNSUPPORTED,
             "%s: not implemented for dtype %d", who, itype);
  HK_REQUIRE(gamma != nullptr, HK_ERR_INVALID, "%s: gamma is required", who);
  HK_REQUIRE(eps >= 0.f, HK_ERR_INVALID, "%s: epsilon must be >= 0", who);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  NormFwdArgs a{};
  a.x = x0; a.residual = residual; a.gamma = gamma; a.beta = beta; a.y = z; a.x_out = x_out;
  int64_t key[3] = {0, 0, 0};
  add_steps(key, x0, x0_steps);
  add_steps(key, residual, residual_steps);
  add_steps(key, z, z_steps);
  add_steps(key, x_out, x_out_steps);
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  walk_steps(w, x0_steps, &a.x_pitch, &a.x_lv);
  walk_steps(w, residual_steps, &a.res_pitch, &a.res_lv);
  walk_steps(w, z_steps, &a.y_pitch, &a.y_lv);
  walk_steps(w, x_out_steps, &a.xout_pitch, &a.xout_lv);
  a.n0 = w.n[0]; a.n1 = w.n[1]; a.n2 = w.n[2]; a.rn = w.rn;
  HK_REQUIRE(rows == 0 || walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)level_rows[0], (long long)level_rows[1], (long long)level_rows[2]);
  a.mean = mu; a.stat = rsigma; a.rows = rows; a.cols = int(cols); a.eps = eps;
  a.is_rms = is_rms_norm ? 1 : 0; a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1;
  return norm_fwd_dispatch(itype, a, as_hip(stream), who);
}

int hk_dropout_add_ln_bwd_strided_rows(int itype, int rtype, int wtype, const void* dz, const int64_t dz_steps[3],
                                       const void* dx_in, const int64_t dx_in_steps[3], const void* x,
                                       const int64_t x_steps[3], const void* mu, const void* rsigma,
                                       const void* gamma, void* dx0, const int64_t dx0_steps[3], void* dresidual,
                                       const int64_t dresidual_steps[3], void* dgamma, void* dbeta,
                                       const int64_t level_rows[3], int64_t cols, int is_rms_norm, void* workspace,
                                       size_t workspace_bytes, hkStream_t stream) {
  const char* who = "hk_dropout_add_ln_bwd_strided_rows";
  HK_REQUIRE(dz_steps && x_steps && dx0_steps && (!dx_in || dx_in_steps) && (!dresidual || dresidual_steps),
             HK_ERR_INVALID, "%s: null steps", who);
  if (!dx_in_steps) dx_in_steps = kNoSteps;
  if (!dresidual_steps) dresidual_steps = kNoSteps;
  int64_t rows = 0;
  int rc = check_levels(level_rows, &rows, who);
  if (rc != HK_OK) return rc;
  HK_REQUIRE(itype == rtype && itype == wtype, HK_ERR_UNSUPPORTED,
             "%s: mixed dtypes (input %d, residual %d, weight %d) are not implemented", who, itype, rtype, wtype);
  HK_REQUIRE(itype == HK_FLOAT32 || itype == HK_BFLOAT16 || itype == HK_FLOAT16, HK_ERR_UNSUPPORTED,
             "%s: not implemented for dtype %d", who, itype);
  HK_REQUIRE(gamma != nullptr, HK_ERR_INVALID, "%s: gamma is required", who);
  HK_REQUIRE(cols >= 0 && cols <= 0x3fffffff, HK_ERR_INVALID, "%s: bad cols", who);
  NormBwdArgs a{};
  a.dy = dz; a.x = x; a.gamma = gamma; a.mean = mu; a.stat = rsigma; a.dx_in = dx_in;
  int64_t key[3] = {0, 0, 0};
  add_steps(key, dz, dz_steps);
  add_steps(key, dx_in, dx_in_steps);
  add_steps(key, x, x_steps);
  add_steps(key, dx0, dx0_steps);
  add_steps(key, dresidual, dresidual_steps);
  const RowWalk w = plan_row_walk(level_rows, key, /*on_grid=*/true);
  walk_steps(w, dz_steps, &a.dy_pitch, &a.dy_lv);
  walk_steps(w, x_steps, &a.x_pitch, &a.x_lv);
  walk_steps(w, dx0_steps, &a.dx_pitch, &a.dx_lv);
  walk_steps(w, dx_in_steps, &a.dxin_pitch, &a.dxin_lv);
  walk_steps(w, dresidual_steps, &a.dres_pitch, &a.dres_lv);
  a.n0 = w.n[0]; a.n1 = w.n[1]; a.n2 = w.n[2]; a.rn = w.rn;
  HK_REQUIRE(rows == 0 || walk_fits_grid(w), HK_ERR_UNSUPPORTED,
             "%s: two of the three levels must hold at most 65535 rows each (got %lld, %lld, %lld)", who,
             (long long)level_rows[0], (long long)level_rows[1], (long long)level_rows[2]);
  a.dx = dx0; a.dres = dresidual; a.rows = rows; a.cols = int(cols); a.eps = 0.f;
  a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1; a.clamp_gamma = 0;
  return norm_bwd_dispatch(itype, a, is_rms_norm ? BWD_RMS : BWD_LN, dgamma, dbeta, workspace, workspace_bytes,
                           as_hip(stream), who);
}

int hk_dropout_add_ln_fwd_pitched(int itype, int rtype, int wtype, const void* x0, int64_t x0_pitch,
                                  const void* residual, int64_t residual_pitch, const void* gamma,
                                  const void* beta, void* z, int64_t z_pitch, void* x_out, int64_t x_out_pitch,
                                  void* mu, void* rsigma, int64_t rows, int64_t cols, float eps,
                                  int is_rms_norm, hkStream_t stream) {
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
  a.x_pitch = x0_pitch; a.res_pitch = residual_pitch; a.y_pitch = z_pitch; a.xout_pitch = x_out_pitch;
  a.mean = mu; a.stat = rsigma; a.rows = rows; a.cols = int(cols); a.eps = eps;
  a.is_rms = is_rms_norm ? 1 : 0; a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1;
  return norm_fwd_dispatch(itype, a, as_hip(stream), "hk_dropout_add_ln_fwd");
}

int hk_dropout_add_ln_fwd(int itype, int rtype, int wtype, const void* x0, const void* residual,
                          const void* gamma, const void* beta, void* z, void* x_out, void* mu,
                          void* rsigma, int64_t rows, int64_t cols, float eps, int is_rms_norm,
                          hkStream_t stream) {
  return hk_dropout_add_ln_fwd_pitched(itype, rtype, wtype, x0, cols, residual, cols, gamma, beta, z, cols, x_out,
                                       cols, mu, rsigma, rows, cols, eps, is_rms_norm, stream);
}

int hk_dropout_add_ln_bwd_pitched(int itype, int rtype, int wtype, const void* dz, int64_t dz_pitch,
                                  const void* dx_in, int64_t dx_in_pitch, const void* x, int64_t x_pitch,
                                  const void* mu, const void* rsigma, const void* gamma, void* dx0,
                                  int64_t dx0_pitch, void* dresidual, int64_t dresidual_pitch, void* dgamma,
                                  void* dbeta, int64_t rows, int64_t cols, int is_rms_norm, void* workspace,
                                  size_t workspace_bytes, hkStream_t stream) {
  HK_REQUIRE(itype == rtype && itype == wtype, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_bwd: mixed dtypes (input %d, residual %d, weight %d) are not implemented",
             itype, rtype, wtype);
  HK_REQUIRE(itype == HK_FLOAT32 || itype == HK_BFLOAT16 || itype == HK_FLOAT16, HK_ERR_UNSUPPORTED,
             "hk_dropout_add_ln_bwd: not implemented for dtype %d", itype);
  HK_REQUIRE(gamma != nullptr, HK_ERR_INVALID, "hk_dropout_add_ln_bwd: gamma is required");
  HK_REQUIRE(cols <= 0x3fffffff, HK_ERR_INVALID, "hk_dropout_add_ln_bwd: cols too large");
  NormBwdArgs a{};
  a.dy = dz; a.x = x; a.gamma = gamma; a.mean = mu; a.stat = rsigma; a.dx_in = dx_in;
  a.dy_pitch = dz_pitch; a.x_pitch = x_pitch; a.dx_pitch = dx0_pitch; a.dxin_pitch = dx_in_pitch;
  a.dres_pitch = dresidual_pitch;
  a.dx = dx0; a.dres = dresidual; a.rows = rows; a.cols = int(cols); a.eps = 0.f;
  a.stat_kind = HK_STAT_RSTD; a.stats_f32 = 1; a.clamp_gamma = 0;
  return norm_bwd_dispatch(itype, a, is_rms_norm ? BWD_RMS : BWD_LN, dgamma, dbeta, workspace,
                           workspace_bytes, as_hip(stream), "hk_dropout_add_ln_bwd");
}

int hk_dropout_add_ln_bwd(int itype, int rtype, int wtype, const void* dz, const void* dx_in,
                          const void* x, const void* mu, const void* rsigma, const void* gamma,
                          void* dx0, void* dresidual, void* dgamma, void* dbeta, int64_t rows,
                          int64_t cols, int is_rms_norm, void* workspace, size_t workspace_bytes,
                          hkStream_t stream) {
  return hk_dropout_add_ln_bwd_pitched(itype, rtype, wtype, dz, cols, dx_in, cols, x, cols, mu, rsigma, gamma, dx0,
                                       cols, dresidual, cols, dgamma, dbeta, rows, cols, is_rms_norm, workspace,
                                       workspace_bytes, stream);
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
