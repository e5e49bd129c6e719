"""ctypes front end of the CPU oracle (oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the bench's
cpu_baseline leg.  Nothing in the product package may import this module.

Every ``oracle_*`` wrapper takes numpy arrays holding values already rounded
to the storage type (as float32) and returns float64 arrays.

The functions written here in numpy (p-norm, batch normalisation, the broadcast
of a reduction's gradient, ...) restate the reference lines their docstrings
cite; each is pinned in tests/test_oracle.py against an independent
implementation (torch float64 and its autograd, numpy broadcasting) and by
closed forms.  No function of this package is left unpinned.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

c_f32p = ctypes.POINTER(ctypes.c_float)
c_f64p = ctypes.POINTER(ctypes.c_double)
c_i64p = ctypes.POINTER(ctypes.c_int64)
c_u16p = ctypes.POINTER(ctypes.c_uint16)


def build(force=False):
    """Compiles oracle.c with the Makefile beside it."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.oracle_bf16_to_f32.restype = ctypes.c_float
        _lib.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_reduce.restype = ctypes.c_int
        _lib.refcpu_num_threads.restype = ctypes.c_int
    return _lib


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _p(a, ptype):
    return None if a is None else a.ctypes.data_as(ptype)


def _i64(v):
    return ctypes.c_int64(int(v))


# ---------------------------------------------------------------------------
# bf16 helpers
# ---------------------------------------------------------------------------
def f32_to_bf16_bits(a):
    a = _f32(a)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16_array(_p(a, c_f32p), _p(out, c_u16p), _i64(a.size))
    return out


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().oracle_bf16_to_f32_array(_p(b, c_u16p), _p(out, c_f32p), _i64(b.size))
    return out


def round_bf16(a):
    """fp32 values rounded to the nearest bf16 (ties to even), as fp32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a))


def round_to(a, dtype):
    """Rounds an array to storage dtype 'fp32' | 'bf16' | 'fp16', returned as fp32."""
    a = np.asarray(a)
    if dtype == "fp32":
        return a.astype(np.float32)
    if dtype == "bf16":
        return round_bf16(a.astype(np.float32))
    if dtype == "fp16":
        return a.astype(np.float16).astype(np.float32)
    raise ValueError(dtype)


# ---------------------------------------------------------------------------
# oracle_* wrappers
# ---------------------------------------------------------------------------
def layernorm_fwd(x, gamma, beta, eps):
    x = _f32(x); gamma = _f32(gamma); beta = _f32(beta)
    rows, cols = x.shape
    y = np.empty((rows, cols)); mean = np.empty(rows); var = np.empty(rows); rstd = np.empty(rows)
    lib().oracle_layernorm_fwd(_p(x, c_f32p), _p(gamma, c_f32p), _p(beta, c_f32p), _i64(rows), _i64(cols),
                               ctypes.c_double(eps), _p(y, c_f64p), _p(mean, c_f64p), _p(var, c_f64p),
                               _p(rstd, c_f64p))
    return y, mean, var, rstd


def layernorm_bwd(dy, x, gamma, mean, rstd, eps=0.0, clamp_gamma=False):
    dy = _f32(dy); x = _f32(x); gamma = _f32(gamma)
    mean = np.ascontiguousarray(mean, dtype=np.float64)
    rstd = np.ascontiguousarray(rstd, dtype=np.float64)
    rows, cols = x.shape
    dx = np.empty((rows, cols)); dg = np.empty(cols); db = np.empty(cols)
    lib().oracle_layernorm_bwd(_p(dy, c_f32p), _p(x, c_f32p), _p(gamma, c_f32p), _p(mean, c_f64p),
                               _p(rstd, c_f64p), _i64(rows), _i64(cols), ctypes.c_double(eps),
                               ctypes.c_int(int(clamp_gamma)), _p(dx, c_f64p), _p(dg, c_f64p), _p(db, c_f64p))
    return dx, dg, db


def layernorm_bwd_memeff(dy, y, gamma, beta, rstd, eps):
    dy = _f32(dy); y = _f32(y); gamma = _f32(gamma); beta = _f32(beta)
    rstd = np.ascontiguousarray(rstd, dtype=np.float64)
    rows, cols = y.shape
    dx = np.empty((rows, cols)); dg = np.empty(cols); db = np.empty(cols)
    lib().oracle_layernorm_bwd_memeff(_p(dy, c_f32p), _p(y, c_f32p), _p(gamma, c_f32p), _p(beta, c_f32p),
                                      _p(rstd, c_f64p), _i64(rows), _i64(cols), ctypes.c_double(eps),
                                      _p(dx, c_f64p), _p(dg, c_f64p), _p(db, c_f64p))
    return dx, dg, db


def dropout_add_ln_fwd(x0, residual, gamma, beta, eps, is_rms):
    x0 = _f32(x0); residual = _f32(residual); gamma = _f32(gamma); beta = _f32(beta)
    rows, cols = x0.shape
    z = np.empty((rows, cols)); xo = np.empty((rows, cols)); mu = np.empty(rows); rs = np.empty(rows)
    lib().oracle_dropout_add_ln_fwd(_p(x0, c_f32p), _p(residual, c_f32p), _p(gamma, c_f32p), _p(beta, c_f32p),
                                    _i64(rows), _i64(cols), ctypes.c_double(eps), ctypes.c_int(int(is_rms)),
                                    _p(z, c_f64p), _p(xo, c_f64p), _p(mu, c_f64p), _p(rs, c_f64p))
    return z, xo, mu, rs


def dropout_add_ln_bwd(dz, dx_in, x, mu, rs, gamma, is_rms):
    dz = _f32(dz); dx_in = _f32(dx_in); x = _f32(x); gamma = _f32(gamma)
    mu = np.ascontiguousarray(mu, dtype=np.float64); rs = np.ascontiguousarray(rs, dtype=np.float64)
    rows, cols = x.shape
    dx = np.empty((rows, cols)); dg = np.empty(cols); db = np.empty(cols)
    lib().oracle_dropout_add_ln_bwd(_p(dz, c_f32p), _p(dx_in, c_f32p), _p(x, c_f32p), _p(mu, c_f64p),
                                    _p(rs, c_f64p), _p(gamma, c_f32p), _i64(rows), _i64(cols),
                                    ctypes.c_int(int(is_rms)), _p(dx, c_f64p), _p(dg, c_f64p), _p(db, c_f64p))
    return dx, dg, db


def softmax_fwd(x, dim=-1):
    x = _f32(x)
    dim = dim % x.ndim
    outer = int(np.prod(x.shape[:dim], dtype=np.int64)); inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    y = np.empty(x.shape)
    lib().oracle_softmax_fwd(_p(x, c_f32p), _i64(outer), _i64(x.shape[dim]), _i64(inner), _p(y, c_f64p))
    return y


def softmax_bwd(y, dy, dim=-1):
    y = _f32(y); dy = _f32(dy)
    dim = dim % y.ndim
    outer = int(np.prod(y.shape[:dim], dtype=np.int64)); inner = int(np.prod(y.shape[dim + 1:], dtype=np.int64))
    dx = np.empty(y.shape)
    lib().oracle_softmax_bwd(_p(y, c_f32p), _p(dy, c_f32p), _i64(outer), _i64(y.shape[dim]), _i64(inner),
                             _p(dx, c_f64p))
    return dx


def sce_sparse_fwd(x, labels, ignored_index):
    x = _f32(x); labels = np.ascontiguousarray(labels, dtype=np.int64)
    rows, cols = x.shape
    loss = np.empty(rows)
    lib().oracle_sce_sparse_fwd(_p(x, c_f32p), _p(labels, c_i64p), _i64(rows), _i64(cols), _i64(ignored_index),
                                _p(loss, c_f64p))
    return loss


def sce_sparse_bwd(x, labels, grad_loss, ignored_index):
    x = _f32(x); labels = np.ascontiguousarray(labels, dtype=np.int64); grad_loss = _f32(grad_loss)
    rows, cols = x.shape
    dx = np.empty((rows, cols))
    lib().oracle_sce_sparse_bwd(_p(x, c_f32p), _p(labels, c_i64p), _p(grad_loss, c_f32p), _i64(rows), _i64(cols),
                                _i64(ignored_index), _p(dx, c_f64p))
    return dx


def sce_dense_fwd(x, labels):
    x = _f32(x); labels = _f32(labels)
    rows, cols = x.shape
    loss = np.empty(rows)
    lib().oracle_sce_dense_fwd(_p(x, c_f32p), _p(labels, c_f32p), _i64(rows), _i64(cols), _p(loss, c_f64p))
    return loss


def sce_dense_bwd(x, labels, grad_loss):
    x = _f32(x); labels = _f32(labels); grad_loss = _f32(grad_loss)
    rows, cols = x.shape
    dx = np.empty((rows, cols))
    lib().oracle_sce_dense_bwd(_p(x, c_f32p), _p(labels, c_f32p), _p(grad_loss, c_f32p), _i64(rows), _i64(cols),
                               _p(dx, c_f64p))
    return dx


def reduce(x, axes, op="sum", mean_mode=0):
    """Sum / mean of a (possibly strided) numpy array over `axes` (already in
    [0, ndim)); returns the dense float64 result with kept dims in order."""
    x = np.asarray(x)
    xd = x.astype(np.float64)  # contiguous copy; strided layouts are exercised through `strided_reduce`
    return strided_reduce(xd, xd.shape, [s // 8 for s in xd.strides], axes, op, mean_mode)


def strided_reduce(buf, shape, strides, axes, op="sum", mean_mode=0):
    buf = np.ascontiguousarray(buf, dtype=np.float64)
    ndim = len(shape)
    sh = (ctypes.c_int64 * max(ndim, 1))(*shape)
    st = (ctypes.c_int64 * max(ndim, 1))(*strides)
    ax = (ctypes.c_int64 * max(len(axes), 1))(*axes)
    red = set(axes)
    out_shape = [shape[d] for d in range(ndim) if d not in red]
    out = np.empty(int(np.prod(out_shape, dtype=np.int64)) if out_shape else 1)
    rc = lib().oracle_reduce(_p(buf.reshape(-1), c_f64p), ctypes.c_int(ndim), sh, st, ctypes.c_int(len(axes)), ax,
                             ctypes.c_int({"sum": 0, "mean": 1, "max": 2, "min": 3, "prod": 4}[op]), ctypes.c_int(mean_mode), _p(out, c_f64p))
    if rc != 0:
        raise ValueError("oracle_reduce: bad arguments")
    return out.reshape(out_shape if out_shape else [1])


def nll_loss_fwd(pred, labels):
    """loss[r] = -pred[r, label[r]], 0 for a label outside [0, cols)
    (hetu/impl/kernel/NLLLoss.cu:8-22).  Plain numpy: a gather has no arithmetic to restate in C."""
    pred = np.asarray(pred, dtype=np.float64)
    rows, cols = pred.shape
    lab = np.asarray(labels, dtype=np.int64)
    ok = (lab >= 0) & (lab < cols)
    out = np.zeros(rows)
    out[ok] = -pred[np.arange(rows)[ok], lab[ok]]
    return out


def nll_loss_bwd(labels, grad_loss, cols):
    """out[r, c] = -grad_loss[r] * cols at c = label[r] (if inside [0, cols)), 0 elsewhere
    (hetu/impl/kernel/NLLLoss.cu:24-41: the array is cleared first, :116, and the factor cols is the reference's)."""
    lab = np.asarray(labels, dtype=np.int64)
    g = np.asarray(grad_loss, dtype=np.float64)
    rows = lab.shape[0]
    out = np.zeros((rows, cols))
    ok = (lab >= 0) & (lab < cols)
    out[np.arange(rows)[ok], lab[ok]] = -g[ok] * cols
    return out


def norm_p_fwd(x, dim, p):
    """(sum_k |x|^p)^(1/p) over `dim` (norm_kernel, hetu/impl/kernel/Norm1.cu:17-56), float64."""
    x = np.asarray(x, dtype=np.float64)
    return (np.abs(x) ** p).sum(axis=dim) ** (1.0 / p)


def norm_p_bwd(x, norm, grad, dim, p):
    """norm_gradient_kernel (Norm1.cu:59-97): p = 1: sign(x) g; p = 2: g x / n; p > 2: x |x|^(p-2) g / n^(p-1);
    0 where the norm is 0 (p >= 2)."""
    x = np.asarray(x, dtype=np.float64)
    n = np.expand_dims(np.asarray(norm, dtype=np.float64), dim)
    g = np.expand_dims(np.asarray(grad, dtype=np.float64), dim)
    if p == 1:
        return np.sign(x) * g
    safe = np.where(n == 0, 1.0, n)
    if p == 2:
        out = g * x / safe
    else:
        out = x * np.abs(x) ** (p - 2) * g / safe ** (p - 1)
    return np.where(n == 0, 0.0, out)


def broadcast_shape(x, out_shape, add_axes=(), const_value=None):
    """broadcast_shape_kernel / broadcast_shape_mul_kernel with the host set-up of BroadcastShapeCuda
    (hetu/impl/kernel/BroadcastShape.cu:11-28, 44-68, 101-117): per output dimension an input extent in_dims[i]
    (1 where the input is laid over a dimension it lacks or broadcasts), and for every output element the flat
    input index  i_ind = sum over dimensions of (in_dims[i] > 1) * coordinate, in row-major order of in_dims.
    Index arithmetic as the kernel does it, one output element at a time; float64 product."""
    x = np.asarray(x)
    out_nd, diff = len(out_shape), len(out_shape) - x.ndim
    if not add_axes:
        in_dims = [1 if i < diff else x.shape[i - diff] for i in range(out_nd)]
    else:
        in_dims = [0] * out_nd
        for i in range(diff):
            in_dims[add_axes[i]] = 1
        o_ind = 0
        for i in range(x.ndim):
            while in_dims[o_ind] == 1:
                o_ind += 1
            in_dims[o_ind] = x.shape[i]
            o_ind += 1
    out_strides = [int(np.prod(out_shape[i + 1:], dtype=np.int64)) for i in range(out_nd)]
    flat = x.reshape(-1)
    size = int(np.prod(out_shape, dtype=np.int64))
    out = np.empty(size, dtype=np.float64)
    for idx in range(size):
        i_ind, temp = 0, idx
        for i in range(out_nd):
            i_ind = i_ind * in_dims[i] + (temp // out_strides[i] if in_dims[i] > 1 else 0)
            temp %= out_strides[i]
        out[idx] = float(flat[i_ind]) * (1.0 if const_value is None else float(const_value))
    return out.reshape(out_shape)


def batch_norm_fwd(x, scale, bias, running_mean, running_var, momentum, eps):
    """Spatial batch normalisation in training mode as cuDNN documents it for
    cudnnBatchNormalizationForwardTraining(CUDNN_BATCHNORM_SPATIAL) (called at
    hetu/impl/kernel/BatchNorm.cu:55-70; cuDNN itself is not among the reference's sources): statistics per
    channel over every other dimension, biased variance in y, unbiased variance into the running average,
    inverse standard deviation saved.  Returns y, new running mean, new running var, save_mean, save_invstd."""
    x = np.asarray(x, dtype=np.float64)
    axes = tuple(i for i in range(x.ndim) if i != 1)
    m = x.size // x.shape[1]
    mean = x.mean(axis=axes)
    var = x.var(axis=axes)
    shape = [1, -1] + [1] * (x.ndim - 2)
    invstd = 1.0 / np.sqrt(var + eps)
    y = (x - mean.reshape(shape)) * (invstd * np.asarray(scale, np.float64)).reshape(shape) \
        + np.asarray(bias, np.float64).reshape(shape)
    unbiased = var * m / (m - 1) if m > 1 else var
    rm = (1 - momentum) * np.asarray(running_mean, np.float64) + momentum * mean
    rv = (1 - momentum) * np.asarray(running_var, np.float64) + momentum * unbiased
    return y, rm, rv, mean, invstd


def batch_norm_bwd(dy, x, scale, save_mean, save_invstd):
    """cudnnBatchNormalizationBackward (BatchNorm.cu:139-153): dscale = sum dy xhat, dbias = sum dy,
    dx = scale invstd (dy - dbias / m - xhat dscale / m)."""
    dy = np.asarray(dy, dtype=np.float64); x = np.asarray(x, dtype=np.float64)
    axes = tuple(i for i in range(x.ndim) if i != 1)
    m = x.size // x.shape[1]
    shape = [1, -1] + [1] * (x.ndim - 2)
    mean = np.asarray(save_mean, np.float64).reshape(shape)
    invstd = np.asarray(save_invstd, np.float64).reshape(shape)
    xhat = (x - mean) * invstd
    dscale = (dy * xhat).sum(axis=axes)
    dbias = dy.sum(axis=axes)
    dx = np.asarray(scale, np.float64).reshape(shape) * invstd * (dy - dbias.reshape(shape) / m
                                                                    - xhat * dscale.reshape(shape) / m)
    return dx, dscale, dbias
