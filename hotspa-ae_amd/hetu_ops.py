"""ctypes bindings of include/hetu_ops_c.h: the C++ operator layer
(libhetu_rowwise.so) called with torch tensors as borrowed arrays.

Errors of the C++ layer come back as Python exceptions named after the C++
ones (AssertionError_, NotImplemented_, ValueError_, RuntimeError_).
"""
import ctypes
import os

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "lib", "libhetu_rowwise.so")
_lib = None

MAX_NDIM = 8
RED = {"sum": 0, "mean": 1, "max": 2, "min": 3, "prod": 4, "none": 5}
DEFAULT_STREAM = 1   # hetu::kComputingStream


class HetuError(RuntimeError):
    kind = "other"


class AssertionError_(HetuError):
    kind = "assertion_error"


class NotImplemented_(HetuError):
    kind = "not_implemented"


class ValueError_(HetuError):
    kind = "value_error"


class RuntimeError_(HetuError):
    kind = "runtime_error"


class BadAlloc_(HetuError):
    kind = "bad_alloc"


_KINDS = {1: AssertionError_, 2: NotImplemented_, 3: ValueError_, 4: RuntimeError_, 5: BadAlloc_}


class HtArray(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.c_int64 * MAX_NDIM), ("stride", ctypes.c_int64 * MAX_NDIM),
                ("device_type", ctypes.c_int32), ("device_index", ctypes.c_int32)]


def lib_path():
    return _LIB


def lib():
    """Loads libhetu_rowwise.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise HetuError("native library %s is missing: run __graft_entry__.build() first" % _LIB)
        capi.lib()   # libhk_rowwise.so first, so the dependency resolves from the same folder
        _lib = ctypes.CDLL(_LIB)
        _lib.ht_last_error.restype = ctypes.c_char_p
    return _lib


def check(rc):
    if rc != 0:
        raise _KINDS.get(rc, HetuError)(lib().ht_last_error().decode("utf-8", "replace"))


def desc(t):
    """HtArray borrowing a torch tensor (None -> NULL = undefined NDArray)."""
    if t is None:
        return None
    assert t.dim() <= MAX_NDIM
    a = HtArray()
    a.data = t.data_ptr()
    a.dtype = capi.dtype_code(t)
    a.ndim = t.dim()
    for i in range(t.dim()):
        a.shape[i] = t.shape[i]
        a.stride[i] = t.stride(i)
    a.device_type = 1 if t.is_cuda else 0
    a.device_index = t.device.index or 0 if t.is_cuda else 0
    a._keep = t
    return a


def _p(a):
    return ctypes.byref(a) if a is not None else None


def _call(name, *args):
    conv = []
    for v in args:
        if isinstance(v, HtArray) or v is None:
            conv.append(_p(v))
        else:
            conv.append(v)
    check(getattr(lib(), name)(*conv))


def _i64(v):
    return ctypes.c_int64(int(v))


def _f(v):
    return ctypes.c_float(float(v))


def _axes(axes):
    axes = list(axes)
    return (ctypes.c_int64 * max(len(axes), 1))(*axes), ctypes.c_int(len(axes))


def stream_sync(stream=DEFAULT_STREAM, device=0):
    check(lib().ht_stream_sync(ctypes.c_int(device), ctypes.c_int(stream)))


def host_stream_sync(stream=DEFAULT_STREAM):
    """Waits for the host stream of that index and raises what a host kernel on it failed with."""
    check(lib().ht_host_stream_sync(ctypes.c_int(stream)))


def set_host_async(on):
    """Host calls return once their work is on its stream (True) or once it has finished (False, the default);
    returns the previous setting.  While on, the caller keeps the arrays alive until host_stream_sync."""
    return bool(lib().ht_set_host_async(ctypes.c_int(int(bool(on)))))


def set_host_threads(n):
    """OpenMP team size of the host twins; returns the size now in force (n <= 0 only asks)."""
    return int(lib().ht_set_host_threads(ctypes.c_int(int(n))))


def synchronize_all():
    check(lib().ht_synchronize_all())


# ---- kernel entry points --------------------------------------------------
def layer_norm(x, scale, bias, mean, var, out, reduce_dims, eps, stream=DEFAULT_STREAM):
    _call("ht_layer_norm", desc(x), desc(scale), desc(bias), desc(mean), desc(var), desc(out), _i64(reduce_dims),
          _f(eps), ctypes.c_int(stream))


def layer_norm_gradient(dy, x, scale, dx, dscale, dbias, mean, var, reduce_dims, eps, stream=DEFAULT_STREAM):
    _call("ht_layer_norm_gradient", desc(dy), desc(x), desc(scale), desc(dx), desc(dscale), desc(dbias), desc(mean),
          desc(var), _i64(reduce_dims), _f(eps), ctypes.c_int(stream))


def fused_layer_norm(x, scale, bias, mean, invvar, out, reduce_dims, eps, stream=DEFAULT_STREAM):
    _call("ht_fused_layer_norm", desc(x), desc(scale), desc(bias), desc(mean), desc(invvar), desc(out),
          _i64(reduce_dims), _f(eps), ctypes.c_int(stream))


def fused_layer_norm_gradient(dy, x_or_y, scale, bias, dx, dscale, dbias, mean, invvar, reduce_dims, eps, inplace,
                              stream=DEFAULT_STREAM):
    _call("ht_fused_layer_norm_gradient", desc(dy), desc(x_or_y), desc(scale), desc(bias), desc(dx), desc(dscale),
          desc(dbias), desc(mean), desc(invvar), _i64(reduce_dims), _f(eps), ctypes.c_int(int(inplace)),
          ctypes.c_int(stream))


def dropout_add_ln_fwd(x0, residual, gamma, beta, z, x, mu, rsigma, eps, is_rms_norm, dropout_p=0.0,
                       rowscale=None, colscale=None, residual_in_fp32=False, x0_subset=None, z_subset=None,
                       dmask=None, rowscale_const=1.0, z_numrows=0, stream=DEFAULT_STREAM):
    _call("ht_dropout_add_ln_fwd", desc(x0), desc(residual), desc(gamma), desc(beta), desc(rowscale),
          desc(colscale), desc(x0_subset), desc(z_subset), desc(z), desc(x), desc(dmask), desc(mu), desc(rsigma),
          _f(dropout_p), _f(eps), _f(rowscale_const), _i64(z_numrows), ctypes.c_int(int(residual_in_fp32)),
          ctypes.c_int(int(is_rms_norm)), ctypes.c_int(stream))


def dropout_add_ln_bwd(dz, dx, x, mu, rsigma, gamma, dx0, dresidual, dgamma, dbeta, has_residual, is_rms_norm,
                       dropout_p=0.0, rowscale=None, colscale=None, x0=None, dmask=None, x0_subset=None,
                       z_subset=None, dcolscale=None, rowscale_const=1.0, x0_numrows=0, stream=DEFAULT_STREAM):
    _call("ht_dropout_add_ln_bwd", desc(dz), desc(dx), desc(x), desc(x0), desc(dmask), desc(mu), desc(rsigma),
          desc(gamma), desc(rowscale), desc(colscale), desc(x0_subset), desc(z_subset), desc(dx0),
          desc(dresidual), desc(dgamma), desc(dbeta), desc(dcolscale), _f(dropout_p), _f(rowscale_const),
          _i64(x0_numrows), ctypes.c_int(int(has_residual)), ctypes.c_int(int(is_rms_norm)), ctypes.c_int(stream))


def dropout_add_ln_parallel_residual_fwd(x0, x1, residual, gamma0, beta0, gamma1, beta1, z0, z1, x, dmask0, dmask1,
                                         mu, rsigma, dropout_p, eps, residual_in_fp32=False, is_rms_norm=False,
                                         stream=DEFAULT_STREAM):
    _call("ht_dropout_add_ln_parallel_residual_fwd", desc(x0), desc(x1), desc(residual), desc(gamma0), desc(beta0),
          desc(gamma1), desc(beta1), desc(z0), desc(z1), desc(x), desc(dmask0), desc(dmask1), desc(mu),
          desc(rsigma), _f(dropout_p), _f(eps), ctypes.c_int(int(residual_in_fp32)),
          ctypes.c_int(int(is_rms_norm)), ctypes.c_int(stream))


def dropout_add_ln_parallel_residual_bwd(dz0, dz1, dx, x, dmask0, dmask1, mu, rsigma, gamma0, gamma1, dx0, dx1,
                                         dresidual, dgamma0, dbeta0, dgamma1, dbeta1, dropout_p, has_x1,
                                         has_residual, is_rms_norm=False, stream=DEFAULT_STREAM):
    _call("ht_dropout_add_ln_parallel_residual_bwd", desc(dz0), desc(dz1), desc(dx), desc(x), desc(dmask0),
          desc(dmask1), desc(mu), desc(rsigma), desc(gamma0), desc(gamma1), desc(dx0), desc(dx1), desc(dresidual),
          desc(dgamma0), desc(dbeta0), desc(dgamma1), desc(dbeta1), _f(dropout_p), ctypes.c_int(int(has_x1)),
          ctypes.c_int(int(has_residual)), ctypes.c_int(int(is_rms_norm)), ctypes.c_int(stream))


BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}
UNARY_OPS = {"exp": 0, "log": 1, "neg": 2, "sqrt": 3}


def binary(op, a, b, out, stream=DEFAULT_STREAM):
    _call("ht_binary", ctypes.c_int(BINARY_OPS[op]), desc(a), desc(b), desc(out), ctypes.c_int(stream))


def binary_const(op, x, value, out, stream=DEFAULT_STREAM):
    """AddConst / SubConst (value - x) / MulConst / DivConst (value / x)."""
    _call("ht_binary_const", ctypes.c_int(BINARY_OPS[op]), desc(x), ctypes.c_double(value), desc(out),
          ctypes.c_int(stream))


def unary(op, x, out, stream=DEFAULT_STREAM):
    _call("ht_unary", ctypes.c_int(UNARY_OPS[op]), desc(x), desc(out), ctypes.c_int(stream))


def ndarray_binary(op, a, b, out=None, in_place=False, stream=DEFAULT_STREAM):
    _call("ht_ndarray_binary", ctypes.c_int(BINARY_OPS[op]), desc(a), desc(b), desc(out),
          ctypes.c_int(int(in_place)), ctypes.c_int(stream))


def ndarray_unary(op, x, out=None, in_place=False, stream=DEFAULT_STREAM):
    _call("ht_ndarray_unary", ctypes.c_int(UNARY_OPS[op]), desc(x), desc(out), ctypes.c_int(int(in_place)),
          ctypes.c_int(stream))


def vocab_parallel_cross_entropy(logits, labels, vocab_start, vocab_end, ignored_index, picked, lse,
                                 stream=DEFAULT_STREAM):
    _call("ht_vocab_parallel_cross_entropy", desc(logits), desc(labels), _i64(vocab_start), _i64(vocab_end),
          _i64(ignored_index), desc(picked), desc(lse), ctypes.c_int(stream))


def vocab_parallel_cross_entropy_gradient(softmax, labels, vocab_start, vocab_end, ignored_index, grad_loss, out,
                                          stream=DEFAULT_STREAM):
    _call("ht_vocab_parallel_cross_entropy_gradient", desc(softmax), desc(labels), _i64(vocab_start),
          _i64(vocab_end), _i64(ignored_index), desc(grad_loss), desc(out), ctypes.c_int(stream))


def norm(x, out, dim, p, stream=DEFAULT_STREAM):
    _call("ht_norm", desc(x), desc(out), _i64(dim), _i64(p), ctypes.c_int(stream))


def norm_gradient(x, norm_out, grad, dx, dim, p, stream=DEFAULT_STREAM):
    _call("ht_norm_gradient", desc(x), desc(norm_out), desc(grad), desc(dx), _i64(dim), _i64(p), ctypes.c_int(stream))


def ndarray_norm(x, p, dim, keepdim, out, stream=DEFAULT_STREAM):
    _call("ht_ndarray_norm", desc(x), _i64(p), _i64(dim), ctypes.c_int(int(keepdim)), desc(out), ctypes.c_int(stream))


def batch_norm(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean, save_var,
               stream=DEFAULT_STREAM):
    _call("ht_batch_norm", desc(x), desc(scale), desc(bias), desc(y), ctypes.c_double(momentum), ctypes.c_double(eps),
          desc(running_mean), desc(running_var), desc(save_mean), desc(save_var), ctypes.c_int(stream))


def batch_norm_gradient(dy, x, scale, dx, dscale, dbias, eps, save_mean, save_var, stream=DEFAULT_STREAM):
    _call("ht_batch_norm_gradient", desc(dy), desc(x), desc(scale), desc(dx), desc(dscale), desc(dbias),
          ctypes.c_double(eps), desc(save_mean), desc(save_var), ctypes.c_int(stream))


def set_random_seed(seed):
    _call("ht_set_random_seed", ctypes.c_uint64(seed))


def instance_norm(x, mean, var, out, eps, stream=DEFAULT_STREAM):
    _call("ht_instance_norm", desc(x), desc(mean), desc(var), desc(out), _f(eps), ctypes.c_int(stream))


def instance_norm_gradient(dy, x, dx, mean, var, eps, stream=DEFAULT_STREAM):
    _call("ht_instance_norm_gradient", desc(dy), desc(x), desc(dx), desc(mean), desc(var), _f(eps),
          ctypes.c_int(stream))


def softmax(x, out, dim, stream=DEFAULT_STREAM):
    _call("ht_softmax", desc(x), desc(out), _i64(dim), ctypes.c_int(stream))


def softmax_gradient(y, dy, dx, dim, stream=DEFAULT_STREAM):
    _call("ht_softmax_gradient", desc(y), desc(dy), desc(dx), _i64(dim), ctypes.c_int(stream))


def softmax_cross_entropy(pred, label, loss, stream=DEFAULT_STREAM):
    _call("ht_softmax_cross_entropy", desc(pred), desc(label), desc(loss), ctypes.c_int(stream))


def softmax_cross_entropy_gradient(pred, label, grad_loss, out, stream=DEFAULT_STREAM):
    _call("ht_softmax_cross_entropy_gradient", desc(pred), desc(label), desc(grad_loss), desc(out),
          ctypes.c_int(stream))


def softmax_cross_entropy_sparse(pred, label, loss, ignored_index, stream=DEFAULT_STREAM):
    _call("ht_softmax_cross_entropy_sparse", desc(pred), desc(label), desc(loss), _i64(ignored_index),
          ctypes.c_int(stream))


def softmax_cross_entropy_sparse_gradient(pred, label, grad_loss, out, ignored_index, stream=DEFAULT_STREAM):
    _call("ht_softmax_cross_entropy_sparse_gradient", desc(pred), desc(label), desc(grad_loss), desc(out),
          _i64(ignored_index), ctypes.c_int(stream))


def nll_loss(pred, label, loss, stream=DEFAULT_STREAM):
    _call("ht_nll_loss", desc(pred), desc(label), desc(loss), ctypes.c_int(stream))


def nll_loss_gradient(pred, label, grad_loss, out, stream=DEFAULT_STREAM):
    _call("ht_nll_loss_gradient", desc(pred), desc(label), desc(grad_loss), desc(out), ctypes.c_int(stream))


def reduce(x, out, axes, red_type, stream=DEFAULT_STREAM):
    ax, n = _axes(axes)
    _call("ht_reduce", desc(x), desc(out), ax, n, ctypes.c_int(RED[red_type]), ctypes.c_int(stream))


# ---- NDArray statics ------------------------------------------------------
def ndarray_reduce(x, red_type, axes, keepdims, out, stream=DEFAULT_STREAM):
    ax, n = _axes(axes)
    _call("ht_ndarray_reduce", desc(x), ctypes.c_int(RED[red_type]), ax, n, ctypes.c_int(int(keepdims)), desc(out),
          ctypes.c_int(stream))


def ndarray_softmax(x, dim, out, stream=DEFAULT_STREAM):
    _call("ht_ndarray_softmax", desc(x), _i64(dim), desc(out), ctypes.c_int(stream))


def ndarray_layernorm(x, scale, bias, normalized_ndim, eps, fused, out, mean=None, var=None,
                      stream=DEFAULT_STREAM):
    _call("ht_ndarray_layernorm", desc(x), desc(scale), desc(bias), ctypes.c_int(normalized_ndim),
          ctypes.c_double(eps), ctypes.c_int(int(fused)), desc(out), desc(mean), desc(var), ctypes.c_int(stream))


def ndarray_sceloss(preds, labels, out, reduction="mean", ignored_index=None, stream=DEFAULT_STREAM):
    sparse = ignored_index is not None
    _call("ht_ndarray_sceloss", desc(preds), desc(labels), ctypes.c_int(int(sparse)),
          _i64(ignored_index if sparse else 0), ctypes.c_int(RED[reduction]), desc(out), ctypes.c_int(stream))


# ---- gradients of the reductions and of the reduced losses ----------------
def broadcast_shape(x, out, add_axes=(), const_value=None, stream=DEFAULT_STREAM):
    """BroadcastShapeCuda, or BroadcastShapeMulCuda when const_value is given."""
    ax, n = _axes(list(add_axes))
    _call("ht_broadcast_shape", desc(x), ctypes.c_int(int(const_value is not None)),
          ctypes.c_double(0.0 if const_value is None else const_value), desc(out), ax, n, ctypes.c_int(stream))


def reduce_gradient(grad_output, out, reduction, axes, keepdims, stream=DEFAULT_STREAM):
    ax, n = _axes(list(axes))
    keep = [keepdims] if isinstance(keepdims, bool) else list(keepdims)
    karr = (ctypes.c_int * max(len(keep), 1))(*[int(k) for k in keep])
    _call("ht_reduce_gradient", desc(grad_output), ctypes.c_int(RED[reduction]), ax, n, karr,
          ctypes.c_int(len(keep)), desc(out), ctypes.c_int(stream))


def sceloss_gradient(preds, labels, grad_output, out, reduction="mean", ignored_index=None, fused=True,
                     stream=DEFAULT_STREAM):
    sparse = ignored_index is not None
    _call("ht_sceloss_gradient", desc(preds), desc(labels), desc(grad_output), ctypes.c_int(int(sparse)),
          _i64(ignored_index if sparse else 0), ctypes.c_int(RED[reduction]), ctypes.c_int(int(fused)), desc(out),
          ctypes.c_int(stream))


# ---- device memory pool ---------------------------------------------------
class PoolBlock:
    def __init__(self, ptr, ident, size, device):
        self.ptr, self.id, self.size, self.device = ptr, ident, size, device


def pool_alloc(nbytes, stream=DEFAULT_STREAM, device=0):
    ptr, ident, granted = ctypes.c_void_p(), ctypes.c_uint64(), ctypes.c_size_t()
    check(lib().ht_pool_alloc(ctypes.c_int(device), ctypes.c_size_t(nbytes), ctypes.c_int(stream),
                              ctypes.byref(ptr), ctypes.byref(ident), ctypes.byref(granted)))
    return PoolBlock(ptr.value or 0, ident.value, granted.value, device)


def pool_free(block):
    check(lib().ht_pool_free(ctypes.c_int(block.device), ctypes.c_void_p(block.ptr), ctypes.c_uint64(block.id),
                             ctypes.c_size_t(block.size)))


def pool_mark_used(block, stream):
    check(lib().ht_pool_mark_used(ctypes.c_int(block.device), ctypes.c_void_p(block.ptr), ctypes.c_uint64(block.id),
                                  ctypes.c_size_t(block.size), ctypes.c_int(stream)))


def pool_empty_cache(device=0):
    check(lib().ht_pool_empty_cache(ctypes.c_int(device)))


_STAT_NAMES = ["allocated", "peak_allocated", "reserved", "peak_reserved", "alloc_cnt", "free_cnt", "mark_cnt",
               "segment_allocs", "segment_frees", "cache_hits", "cross_stream_takes", "parked", "splits", "merges"]


def pool_stats(device=0):
    vals = (ctypes.c_uint64 * len(_STAT_NAMES))()
    check(lib().ht_pool_stats(ctypes.c_int(device), vals, ctypes.c_int(len(_STAT_NAMES))))
    return dict(zip(_STAT_NAMES, [int(v) for v in vals]))
