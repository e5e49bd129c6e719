"""ctypes bindings of include/hk_rowwise.h operating on torch CUDA tensors.

torch is used for device memory and streams only; every computation goes
through the C-ABI entry points.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "lib", "libhk_rowwise.so")
_lib = None

HK_FLOAT16, HK_FLOAT32, HK_FLOAT64, HK_BFLOAT16, HK_INT64 = 5, 6, 7, 8, 4
HK_STAT_VAR, HK_STAT_RSTD = 0, 1
HK_REDUCE_SUM, HK_REDUCE_MEAN, HK_REDUCE_MAX, HK_REDUCE_MIN, HK_REDUCE_PROD = 0, 1, 2, 3, 4
REDUCE_OPS = {"sum": 0, "mean": 1, "max": 2, "min": 3, "prod": 4}

DTYPES = {"uint8": 0, "int8": 1, "int16": 2, "int32": 3, "int64": 4, "fp16": 5, "fp32": 6,
          "fp64": 7, "bf16": 8, "bool": 9}


class HkError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("hk error %d: %s" % (code, message))
        self.code = code


def lib_path():
    return _LIB


_BENCH_LIB = os.path.join(_HERE, "lib", "libhk_bench.so")
_bench_lib = None


def bench_lib():
    """Loads libhk_bench.so (the streaming yardstick of include/hk_bench.h); raises if it has not been built."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(_BENCH_LIB):
            raise HkError(-100, "native library %s is missing: run __graft_entry__.build() first" % _BENCH_LIB)
        _bench_lib = ctypes.CDLL(_BENCH_LIB)
        _bench_lib.hk_bench_last_error.restype = ctypes.c_char_p
    return _bench_lib


def lib():
    """Loads libhk_rowwise.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise HkError(-100, "native library %s is missing: run __graft_entry__.build() "
                                "(or python hotspa-ae_amd/build.py) first" % _LIB)
        _lib = ctypes.CDLL(_LIB)
        _lib.hk_last_error.restype = ctypes.c_char_p
        _lib.hk_version.restype = ctypes.c_char_p
        _lib.hk_tune_keys.restype = ctypes.c_char_p
    return _lib


def check(rc):
    if rc != 0:
        raise HkError(rc, lib().hk_last_error().decode("utf-8", "replace"))


def dtype_code(t):
    import torch
    return {torch.float16: 5, torch.float32: 6, torch.float64: 7, torch.bfloat16: 8, torch.int64: 4,
            torch.int32: 3, torch.int16: 2, torch.int8: 1, torch.uint8: 0, torch.bool: 9}[t.dtype]


def torch_dtype(name):
    import torch
    return {"fp16": torch.float16, "fp32": torch.float32, "fp64": torch.float64, "bf16": torch.bfloat16,
            "int64": torch.int64, "int32": torch.int32, "int16": torch.int16, "int8": torch.int8,
            "uint8": torch.uint8}[name]


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def current_stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _i64(v):
    return ctypes.c_int64(int(v))


def _arr(vals):
    vals = list(vals)
    return (ctypes.c_int64 * max(len(vals), 1))(*vals)


def tune_set(key, value):
    check(lib().hk_tune_set(key.encode(), ctypes.c_int(int(value))))


class Event:
    """hipEvent through the C-ABI, recorded on torch's current stream."""

    def __init__(self):
        self.h = ctypes.c_void_p()
        check(lib().hk_event_create(ctypes.byref(self.h), ctypes.c_int(1)))

    def record(self, stream=None):
        check(lib().hk_event_record(self.h, stream if stream is not None else current_stream()))

    def sync(self):
        check(lib().hk_event_sync(self.h))

    def elapsed_ns_since(self, start):
        ns = ctypes.c_int64()
        check(lib().hk_event_elapsed_ns(start.h, self.h, ctypes.byref(ns)))
        return ns.value

    def __del__(self):
        try:
            if self.h:
                lib().hk_event_destroy(self.h)
        except Exception:
            pass


# ---------------------------------------------------------------------------
# operators: tensors are torch CUDA tensors, already allocated; dense, or 2-D views whose rows lie a constant
# pitch apart (a column slice of a wider tensor), which go to the *_pitched entry points as they are
# ---------------------------------------------------------------------------
def _pitch(t, cols):
    """Row pitch, in elements, of a [rows, cols] operand: its row stride when it is a 2-D view with a unit-stride
    last dimension, cols when it is dense (any number of leading dimensions) or absent."""
    if t is None or t.is_contiguous():
        return cols
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise HkError(-1, "operand must be dense or a 2-D view with a unit-stride last dimension, got shape %s "
                          "strides %s" % (tuple(t.shape), tuple(t.stride())))
    return t.stride(0) if t.shape[0] > 1 else cols


def row_levels(tensors):
    """The joint row levels of same-shaped operands whose last dimension has unit stride: (level_rows, steps) with
    level_rows = [n0, n1, n2] innermost first and steps[k] = the three element steps of operand k (None for an absent
    operand), as the *_strided_rows entry points take them.  Leading dimensions that step together in EVERY operand
    are merged; returns None when more than three levels remain."""
    present = [t for t in tensors if t is not None]
    ref = present[0]
    nd = ref.dim()
    for t in present:
        if tuple(t.shape) != tuple(ref.shape):
            raise HkError(-1, "operands of one call must have one shape, got %s and %s" % (tuple(ref.shape), tuple(t.shape)))
        if nd and t.shape[-1] > 1 and t.stride(-1) != 1:
            raise HkError(-1, "the last dimension must have unit stride, got strides %s" % (tuple(t.stride()),))
    cols = ref.shape[-1] if nd else 1
    levels = []                      # (count, [step of every present operand]), innermost first
    for i in range(nd - 2, -1, -1):
        n = ref.shape[i]
        if n == 1:
            continue
        steps = [t.stride(i) for t in present]
        if levels and all(st == levels[-1][0] * ls for st, ls in zip(steps, levels[-1][1])):
            levels[-1] = (levels[-1][0] * n, levels[-1][1])
        else:
            levels.append((n, steps))
    if len(levels) > 3:
        return None
    while len(levels) < 3:
        levels.append((1, [cols if not levels else 0] * len(present)))
    counts = [l[0] for l in levels]
    out, k = [], 0
    for t in tensors:
        if t is None:
            out.append(None)
        else:
            out.append([levels[0][1][k], levels[1][1][k], levels[2][1][k]])
            k += 1
    return counts, out


def _steps(v):
    return None if v is None else _arr(v)


def _multi_level(tensors):
    """(level_rows, steps) when the operands need the *_strided_rows entry points: some operand is neither dense
    nor a 2-D row-pitched view.  None when the dense / pitched entry points take them (or nothing does)."""
    present = [t for t in tensors if t is not None]
    if all(t.is_contiguous() or t.dim() == 2 for t in present):
        return None
    lv = row_levels(tensors)
    if lv is None:
        raise HkError(-1, "operands need more than three row levels; make them dense first")
    return lv


def layer_norm_fwd(x, gamma, beta, y, mean, stat, eps, stat_kind=HK_STAT_RSTD, stream=None):
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    cols = x.shape[-1]
    lv = _multi_level([x, y])
    if lv is not None:
        counts, (xs, ys) = lv
        check(lib().hk_layer_norm_fwd_strided_rows(dtype_code(x), _ptr(x), _steps(xs), _ptr(gamma), _ptr(beta), _ptr(y),
                                                   _steps(ys), _ptr(mean), _ptr(stat),
                                                   dtype_code(mean if mean is not None else stat),
                                                   ctypes.c_int(stat_kind), _arr(counts), _i64(cols),
                                                   ctypes.c_float(eps),
                                                   stream if stream is not None else current_stream()))
        return
    check(lib().hk_layer_norm_fwd_pitched(dtype_code(x), _ptr(x), _i64(_pitch(x, cols)), _ptr(gamma), _ptr(beta),
                                          _ptr(y), _i64(_pitch(y, cols)), _ptr(mean), _ptr(stat),
                                          dtype_code(mean if mean is not None else stat), ctypes.c_int(stat_kind),
                                          _i64(rows), _i64(cols), ctypes.c_float(eps),
                                          stream if stream is not None else current_stream()))


def norm_bwd_workspace_bytes(dtype, rows, cols):
    n = ctypes.c_size_t()
    check(lib().hk_norm_bwd_workspace_bytes(ctypes.c_int(dtype), _i64(rows), _i64(cols), ctypes.byref(n)))
    return n.value


def _workspace(nbytes, device):
    import torch
    if nbytes == 0:
        return None
    return torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)


def layer_norm_bwd(dy, x_or_y, gamma, beta, mean, stat, dx, dgamma, dbeta, eps, stat_kind=HK_STAT_RSTD,
                   memory_efficient=False, clamp_gamma=False, workspace=None, stream=None):
    cols = dy.shape[-1]
    rows = dy.numel() // cols if dy.numel() else 0
    if workspace is None:
        workspace = _workspace(norm_bwd_workspace_bytes(dtype_code(dy), rows, cols), dy.device)
    wsb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    lv = _multi_level([dy, x_or_y, dx])
    if lv is not None:
        counts, (dys, xs, dxs) = lv
        check(lib().hk_layer_norm_bwd_strided_rows(dtype_code(dy), _ptr(dy), _steps(dys), _ptr(x_or_y), _steps(xs),
                                                   _ptr(gamma), _ptr(beta), _ptr(mean), _ptr(stat), dtype_code(stat),
                                                   ctypes.c_int(stat_kind), _ptr(dx), _steps(dxs), _ptr(dgamma),
                                                   _ptr(dbeta), _arr(counts), _i64(cols), ctypes.c_float(eps),
                                                   ctypes.c_int(int(memory_efficient)), ctypes.c_int(int(clamp_gamma)),
                                                   _ptr(workspace), ctypes.c_size_t(wsb),
                                                   stream if stream is not None else current_stream()))
        return workspace
    check(lib().hk_layer_norm_bwd_pitched(dtype_code(dy), _ptr(dy), _i64(_pitch(dy, cols)), _ptr(x_or_y),
                                          _i64(_pitch(x_or_y, cols)), _ptr(gamma), _ptr(beta), _ptr(mean),
                                          _ptr(stat), dtype_code(stat), ctypes.c_int(stat_kind), _ptr(dx),
                                          _i64(_pitch(dx, cols)), _ptr(dgamma), _ptr(dbeta), _i64(rows), _i64(cols),
                                          ctypes.c_float(eps), ctypes.c_int(int(memory_efficient)),
                                          ctypes.c_int(int(clamp_gamma)), _ptr(workspace), ctypes.c_size_t(wsb),
                                          stream if stream is not None else current_stream()))
    return workspace


def dropout_add_ln_fwd(x0, residual, gamma, beta, z, x_out, mu, rsigma, eps, is_rms, stream=None):
    cols = x0.shape[-1]
    rows = x0.numel() // cols if x0.numel() else 0
    rtype = dtype_code(residual) if residual is not None else dtype_code(x0)
    lv = _multi_level([x0, residual, z, x_out])
    if lv is not None:
        counts, (xs, rs_, zs, xos) = lv
        check(lib().hk_dropout_add_ln_fwd_strided_rows(dtype_code(x0), rtype, dtype_code(gamma), _ptr(x0), _steps(xs),
                                                       _ptr(residual), _steps(rs_), _ptr(gamma), _ptr(beta), _ptr(z),
                                                       _steps(zs), _ptr(x_out), _steps(xos), _ptr(mu), _ptr(rsigma),
                                                       _arr(counts), _i64(cols), ctypes.c_float(eps),
                                                       ctypes.c_int(int(is_rms)),
                                                       stream if stream is not None else current_stream()))
        return
    check(lib().hk_dropout_add_ln_fwd_pitched(dtype_code(x0), rtype, dtype_code(gamma), _ptr(x0),
                                              _i64(_pitch(x0, cols)), _ptr(residual), _i64(_pitch(residual, cols)),
                                              _ptr(gamma), _ptr(beta), _ptr(z), _i64(_pitch(z, cols)), _ptr(x_out),
                                              _i64(_pitch(x_out, cols)), _ptr(mu), _ptr(rsigma), _i64(rows),
                                              _i64(cols), ctypes.c_float(eps), ctypes.c_int(int(is_rms)),
                                              stream if stream is not None else current_stream()))


def dropout_add_ln_bwd(dz, dx_in, x, mu, rsigma, gamma, dx0, dresidual, dgamma, dbeta, is_rms,
                       workspace=None, stream=None):
    cols = x.shape[-1]
    rows = x.numel() // cols if x.numel() else 0
    if workspace is None:
        workspace = _workspace(norm_bwd_workspace_bytes(dtype_code(dz), rows, cols), dz.device)
    wsb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    lv = _multi_level([dz, dx_in, x, dx0, dresidual])
    if lv is not None:
        counts, (dzs, dis, xs, dxs, drs) = lv
        check(lib().hk_dropout_add_ln_bwd_strided_rows(dtype_code(dz), dtype_code(x), dtype_code(gamma), _ptr(dz),
                                                       _steps(dzs), _ptr(dx_in), _steps(dis), _ptr(x), _steps(xs),
                                                       _ptr(mu), _ptr(rsigma), _ptr(gamma), _ptr(dx0), _steps(dxs),
                                                       _ptr(dresidual), _steps(drs), _ptr(dgamma), _ptr(dbeta),
                                                       _arr(counts), _i64(cols), ctypes.c_int(int(is_rms)),
                                                       _ptr(workspace), ctypes.c_size_t(wsb),
                                                       stream if stream is not None else current_stream()))
        return workspace
    check(lib().hk_dropout_add_ln_bwd_pitched(dtype_code(dz), dtype_code(x), dtype_code(gamma), _ptr(dz),
                                              _i64(_pitch(dz, cols)), _ptr(dx_in), _i64(_pitch(dx_in, cols)),
                                              _ptr(x), _i64(_pitch(x, cols)), _ptr(mu), _ptr(rsigma), _ptr(gamma),
                                              _ptr(dx0), _i64(_pitch(dx0, cols)), _ptr(dresidual),
                                              _i64(_pitch(dresidual, cols)), _ptr(dgamma), _ptr(dbeta), _i64(rows),
                                              _i64(cols), ctypes.c_int(int(is_rms)), _ptr(workspace),
                                              ctypes.c_size_t(wsb),
                                              stream if stream is not None else current_stream()))
    return workspace


def dropout_add_ln_bwd_static(dz, dx_in, x, mu, rsigma, gamma, dx0, dresidual, dgamma, dbeta, is_rms, stream=None):
    """hk_dropout_add_ln_bwd_static: the same backward with its partials in the library's own static array;
    nothing is allocated, here or inside."""
    rows, cols = x.shape
    check(lib().hk_dropout_add_ln_bwd_static(dtype_code(dz), dtype_code(x), dtype_code(gamma), _ptr(dz),
                                             _ptr(dx_in), _ptr(x), _ptr(mu), _ptr(rsigma), _ptr(gamma), _ptr(dx0),
                                             _ptr(dresidual), _ptr(dgamma), _ptr(dbeta), _i64(rows), _i64(cols),
                                             ctypes.c_int(int(is_rms)),
                                             stream if stream is not None else current_stream()))


class DropoutAddLnFwdParams(ctypes.Structure):
    """hkDropoutAddLnFwdParams of include/hk_rowwise.h"""
    _fields_ = [("itype", ctypes.c_int), ("rtype", ctypes.c_int), ("wtype", ctypes.c_int),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("x0_numrows", ctypes.c_int64),
                ("z_numrows", ctypes.c_int64)] + \
               [(n, ctypes.c_void_p) for n in ("x0", "x1", "residual", "gamma", "beta", "gamma1", "beta1",
                                               "rowscale", "colscale", "x0_subset", "z_subset", "z", "z1", "x",
                                               "dmask", "dmask1", "mu", "rs")] + \
               [("dropout_p", ctypes.c_float), ("epsilon", ctypes.c_float), ("rowscale_const", ctypes.c_float),
                ("is_rms_norm", ctypes.c_int), ("seed", ctypes.c_uint64), ("offset", ctypes.c_uint64)]


class DropoutAddLnBwdParams(ctypes.Structure):
    """hkDropoutAddLnBwdParams of include/hk_rowwise.h"""
    _fields_ = [("itype", ctypes.c_int), ("rtype", ctypes.c_int), ("wtype", ctypes.c_int),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("x0_numrows", ctypes.c_int64),
                ("z_numrows", ctypes.c_int64)] + \
               [(n, ctypes.c_void_p) for n in ("dz", "dz1", "dx", "x", "x0", "dmask", "dmask1", "mu", "rs", "gamma",
                                               "gamma1", "rowscale", "colscale", "x0_subset", "z_subset", "dx0",
                                               "dx1", "dresidual", "dgamma", "dbeta", "dgamma1", "dbeta1",
                                               "dcolscale", "workspace")] + \
               [("workspace_bytes", ctypes.c_size_t), ("dropout_p", ctypes.c_float),
                ("rowscale_const", ctypes.c_float), ("is_rms_norm", ctypes.c_int)]


def _addr(t):
    return None if t is None else t.data_ptr()


def dropout_add_ln_fwd_ex(x0, gamma, z, mu, rs, *, x1=None, residual=None, beta=None, gamma1=None, beta1=None,
                          rowscale=None, colscale=None, x0_subset=None, z_subset=None, z1=None, x=None,
                          dmask=None, dmask1=None, dropout_p=0.0, eps=1e-5, rowscale_const=1.0, is_rms=False,
                          seed=0, offset=0, rtype=None, stream=None):
    """hk_dropout_add_ln_fwd_ex on torch tensors; rows is the length of the subsets when they are given.
    rtype (a dtype code) names the residual type when neither residual nor x is passed."""
    p = DropoutAddLnFwdParams()
    p.itype = dtype_code(x0)
    p.wtype = dtype_code(gamma)
    if residual is not None:
        p.rtype = dtype_code(residual)
    elif x is not None:
        p.rtype = dtype_code(x)
    else:
        p.rtype = p.itype if rtype is None else rtype
    p.cols = x0.shape[1]
    p.rows = x0.shape[0] if x0_subset is None else x0_subset.numel()
    p.x0_numrows = x0.shape[0]
    p.z_numrows = z.shape[0]
    for name, t in (("x0", x0), ("x1", x1), ("residual", residual), ("gamma", gamma), ("beta", beta),
                    ("gamma1", gamma1), ("beta1", beta1), ("rowscale", rowscale), ("colscale", colscale),
                    ("x0_subset", x0_subset), ("z_subset", z_subset), ("z", z), ("z1", z1), ("x", x),
                    ("dmask", dmask), ("dmask1", dmask1), ("mu", mu), ("rs", rs)):
        setattr(p, name, _addr(t))
    p.dropout_p = dropout_p; p.epsilon = eps; p.rowscale_const = rowscale_const
    p.is_rms_norm = int(is_rms); p.seed = seed; p.offset = offset
    check(lib().hk_dropout_add_ln_fwd_ex(ctypes.byref(p), stream if stream is not None else current_stream()))


def dropout_add_ln_bwd_ex(dz, x, mu, rs, gamma, dx0, *, dz1=None, dx=None, x0=None, dmask=None, dmask1=None,
                          gamma1=None, rowscale=None, colscale=None, x0_subset=None, z_subset=None, dx1=None,
                          dresidual=None, dgamma=None, dbeta=None, dgamma1=None, dbeta1=None, dcolscale=None,
                          dropout_p=0.0, rowscale_const=1.0, is_rms=False, workspace=None, stream=None):
    """hk_dropout_add_ln_bwd_ex on torch tensors; allocates the workspace when none is passed."""
    p = DropoutAddLnBwdParams()
    p.itype = dtype_code(dz); p.rtype = dtype_code(x); p.wtype = dtype_code(gamma)
    p.rows, p.cols = x.shape
    p.x0_numrows = dx0.shape[0]
    p.z_numrows = dz.shape[0]
    for name, t in (("dz", dz), ("dz1", dz1), ("dx", dx), ("x", x), ("x0", x0), ("dmask", dmask),
                    ("dmask1", dmask1), ("mu", mu), ("rs", rs), ("gamma", gamma), ("gamma1", gamma1),
                    ("rowscale", rowscale), ("colscale", colscale), ("x0_subset", x0_subset),
                    ("z_subset", z_subset), ("dx0", dx0), ("dx1", dx1), ("dresidual", dresidual),
                    ("dgamma", dgamma), ("dbeta", dbeta), ("dgamma1", dgamma1), ("dbeta1", dbeta1),
                    ("dcolscale", dcolscale)):
        setattr(p, name, _addr(t))
    p.dropout_p = dropout_p; p.rowscale_const = rowscale_const; p.is_rms_norm = int(is_rms)
    if workspace is None:
        need = ctypes.c_size_t(0)
        check(lib().hk_dropout_add_ln_bwd_ex_workspace_bytes(ctypes.byref(p), ctypes.byref(need)))
        workspace = _workspace(need.value, dz.device)
    p.workspace = _addr(workspace)
    p.workspace_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib().hk_dropout_add_ln_bwd_ex(ctypes.byref(p), stream if stream is not None else current_stream()))
    return workspace


UNARY_OPS = {"exp": 0, "log": 1, "neg": 2, "sqrt": 3}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def unary(op, x, out, stream=None):
    """hk_unary: out = op(x), dense arrays of one dtype (out may be x)."""
    check(lib().hk_unary(UNARY_OPS[op], dtype_code(x), _ptr(x), _ptr(out), _i64(x.numel()),
                         stream if stream is not None else current_stream()))


def binary_const(op, x, scalar, out, scalar_first=False, stream=None):
    """hk_binary_const: out = x op scalar (scalar op x when scalar_first)."""
    check(lib().hk_binary_const(BINARY_OPS[op], dtype_code(x), _ptr(x), ctypes.c_double(scalar),
                                ctypes.c_int(int(scalar_first)), _ptr(out), _i64(x.numel()),
                                stream if stream is not None else current_stream()))


def binary(op, a, b, out, stream=None):
    """hk_binary: out = a op b, broadcasting a and b (any strides) to out's shape; out is dense."""
    shape = list(out.shape)
    sa = list(a.expand(shape).stride())
    sb = list(b.expand(shape).stride())
    check(lib().hk_binary(BINARY_OPS[op], dtype_code(out), _ptr(a), _ptr(b), _ptr(out), ctypes.c_int(len(shape)),
                          _arr(shape), _arr(sa), _arr(sb), stream if stream is not None else current_stream()))


def broadcast(x, out, scalar=None, stream=None):
    """hk_broadcast: out (dense) = x broadcast to out's shape (x.expand(out.shape) must be legal; any strides),
    times `scalar` when given."""
    shape = list(out.shape)
    sx = list(x.expand(shape).stride())
    check(lib().hk_broadcast(dtype_code(out), _ptr(x), ctypes.c_int(int(scalar is not None)),
                             ctypes.c_double(0.0 if scalar is None else scalar), _ptr(out), ctypes.c_int(len(shape)),
                             _arr(shape), _arr(sx), stream if stream is not None else current_stream()))


def vocab_parallel_ce_gather(logits, labels, vocab_start, vocab_end, ignored_index, picked, lse, stream=None):
    rows, cols = logits.shape
    check(lib().hk_vocab_parallel_ce_gather(dtype_code(logits), _ptr(logits), _ptr(labels), _i64(rows), _i64(cols),
                                            _i64(vocab_start), _i64(vocab_end), _i64(ignored_index), _ptr(picked),
                                            _ptr(lse), stream if stream is not None else current_stream()))


def vocab_parallel_ce_bwd(softmax, labels, grad_loss, out, vocab_start, stream=None):
    rows, cols = softmax.shape
    check(lib().hk_vocab_parallel_ce_bwd(dtype_code(softmax), _ptr(softmax), _ptr(labels), _ptr(grad_loss),
                                         _ptr(out), _i64(rows), _i64(cols), _i64(vocab_start),
                                         stream if stream is not None else current_stream()))


def vocab_parallel_ce_stats(logits, labels, stats, vocab_start, ignored_index, stream=None):
    """stats: fp32 [3, rows] (row maximum, sum of exp(x - maximum), picked logit) of this column shard."""
    rows, cols = logits.shape
    check(lib().hk_vocab_parallel_ce_stats(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(stats), _i64(rows),
                                           _i64(cols), _i64(vocab_start), _i64(ignored_index),
                                           stream if stream is not None else current_stream()))


def vocab_parallel_ce_combine(stats, labels, ignored_index, loss, lse, stream=None):
    """stats: fp32 [nshards, 3, rows]; loss (any float dtype) and lse (fp32) are [rows]; either may be None."""
    nshards, _, rows = stats.shape
    code = dtype_code(loss) if loss is not None else HK_FLOAT32
    check(lib().hk_vocab_parallel_ce_combine(code, _ptr(stats), ctypes.c_int(nshards), _ptr(labels),
                                             _i64(ignored_index), _ptr(loss), _ptr(lse), _i64(rows),
                                             stream if stream is not None else current_stream()))


def vocab_parallel_ce_bwd_fused(logits, labels, lse, grad_loss, out, vocab_start, ignored_index, stream=None):
    rows, cols = logits.shape
    check(lib().hk_vocab_parallel_ce_bwd_fused(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(lse),
                                               _ptr(grad_loss), _ptr(out), _i64(rows), _i64(cols),
                                               _i64(vocab_start), _i64(ignored_index),
                                               stream if stream is not None else current_stream()))


def norm(x, out, dim, p, workspace=None, stream=None):
    """hk_norm: p-norm of x (any strided view) over `dim` (already wrapped); out is dense."""
    shape, strides = list(x.shape), list(x.stride())
    if workspace is None:
        workspace = _workspace(reduce_workspace_bytes(dtype_code(x), shape, strides, [dim]), x.device)
    wsb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib().hk_norm(dtype_code(x), _ptr(x), _ptr(out), ctypes.c_int(len(shape)), _arr(shape), _arr(strides),
                        _i64(dim), _i64(p), _ptr(workspace), ctypes.c_size_t(wsb),
                        stream if stream is not None else current_stream()))
    return workspace


def norm_bwd(x, norm_out, grad, out, dim, p, stream=None):
    """hk_norm_bwd on dense tensors; x viewed as [before, x.shape[dim], after]."""
    before, _, after = _odi(list(x.shape), dim)
    check(lib().hk_norm_bwd(dtype_code(x), _ptr(x), _ptr(norm_out), _ptr(grad), _ptr(out), _i64(before),
                            _i64(x.shape[dim]), _i64(after), _i64(p),
                            stream if stream is not None else current_stream()))


def batch_norm_workspace_bytes(x):
    n, c = x.shape[0], x.shape[1]
    hw = x.numel() // max(n * c, 1)
    need = ctypes.c_size_t(0)
    check(lib().hk_batch_norm_workspace_bytes(dtype_code(x), _i64(n), _i64(c), _i64(hw), ctypes.byref(need)))
    return need.value


def _bn_workspace(x, workspace):
    n, c = x.shape[0], x.shape[1]
    hw = x.numel() // max(n * c, 1)
    if workspace is None:
        workspace = _workspace(batch_norm_workspace_bytes(x), x.device)
    return n, c, hw, workspace


def batch_norm_fwd(x, scale, bias, y, momentum, eps, running_mean, running_var, save_mean, save_invstd,
                   workspace=None, stream=None):
    """hk_batch_norm_fwd on a dense [N, C, ...] tensor; allocates the workspace when none is passed."""
    n, c, hw, ws = _bn_workspace(x, workspace)
    wsb = 0 if ws is None else ws.numel() * ws.element_size()
    check(lib().hk_batch_norm_fwd(dtype_code(x), _ptr(x), _ptr(scale), _ptr(bias), _ptr(y), ctypes.c_double(momentum),
                                  ctypes.c_double(eps), _ptr(running_mean), _ptr(running_var), _ptr(save_mean),
                                  _ptr(save_invstd), _i64(n), _i64(c), _i64(hw), _ptr(ws), ctypes.c_size_t(wsb),
                                  stream if stream is not None else current_stream()))


def batch_norm_bwd(dy, x, scale, dx, dscale, dbias, save_mean, save_invstd, workspace=None, stream=None):
    n, c, hw, ws = _bn_workspace(x, workspace)
    wsb = 0 if ws is None else ws.numel() * ws.element_size()
    check(lib().hk_batch_norm_bwd(dtype_code(x), _ptr(dy), _ptr(x), _ptr(scale), _ptr(dx), _ptr(dscale), _ptr(dbias),
                                  _ptr(save_mean), _ptr(save_invstd), _i64(n), _i64(c), _i64(hw), _ptr(ws),
                                  ctypes.c_size_t(wsb), stream if stream is not None else current_stream()))


def _odi(shape, dim):
    dim = dim % len(shape)
    outer = 1
    for s in shape[:dim]:
        outer *= s
    inner = 1
    for s in shape[dim + 1:]:
        inner *= s
    return outer, shape[dim], inner


def softmax_fwd(x, y, dim=-1, stream=None):
    if dim in (-1, x.dim() - 1):
        lv = _multi_level([x, y])
        if lv is not None:
            counts, (xs, ys) = lv
            check(lib().hk_softmax_fwd_strided_rows(dtype_code(x), _ptr(x), _steps(xs), _ptr(y), _steps(ys),
                                                    _arr(counts), _i64(x.shape[-1]),
                                                    stream if stream is not None else current_stream()))
            return
    if x.dim() == 2 and dim in (-1, 1) and not (x.is_contiguous() and y.is_contiguous()):
        rows, cols = x.shape
        check(lib().hk_softmax_fwd_pitched(dtype_code(x), _ptr(x), _i64(_pitch(x, cols)), _ptr(y),
                                           _i64(_pitch(y, cols)), _i64(rows), _i64(cols),
                                           stream if stream is not None else current_stream()))
        return
    o, d, i = _odi(list(x.shape), dim)
    check(lib().hk_softmax_fwd(dtype_code(x), _ptr(x), _ptr(y), _i64(o), _i64(d), _i64(i),
                               stream if stream is not None else current_stream()))


def softmax_bwd(y, dy, dx, dim=-1, stream=None):
    if dim in (-1, y.dim() - 1):
        lv = _multi_level([y, dy, dx])
        if lv is not None:
            counts, (ys, dys, dxs) = lv
            check(lib().hk_softmax_bwd_strided_rows(dtype_code(y), _ptr(y), _steps(ys), _ptr(dy), _steps(dys), _ptr(dx),
                                                    _steps(dxs), _arr(counts), _i64(y.shape[-1]),
                                                    stream if stream is not None else current_stream()))
            return
    if y.dim() == 2 and dim in (-1, 1) and not (y.is_contiguous() and dy.is_contiguous() and dx.is_contiguous()):
        rows, cols = y.shape
        check(lib().hk_softmax_bwd_pitched(dtype_code(y), _ptr(y), _i64(_pitch(y, cols)), _ptr(dy),
                                           _i64(_pitch(dy, cols)), _ptr(dx), _i64(_pitch(dx, cols)), _i64(rows),
                                           _i64(cols), stream if stream is not None else current_stream()))
        return
    o, d, i = _odi(list(y.shape), dim)
    check(lib().hk_softmax_bwd(dtype_code(y), _ptr(y), _ptr(dy), _ptr(dx), _i64(o), _i64(d), _i64(i),
                               stream if stream is not None else current_stream()))


def sce_sparse_fwd(logits, labels, loss, ignored_index, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    lv = _multi_level([logits])
    if lv is not None:
        counts, (xs,) = lv
        check(lib().hk_sce_sparse_fwd_strided_rows(dtype_code(logits), _ptr(logits), _steps(xs), _ptr(labels),
                                                   _ptr(loss), _arr(counts), _i64(cols), _i64(ignored_index),
                                                   stream if stream is not None else current_stream()))
        return
    check(lib().hk_sce_sparse_fwd_pitched(dtype_code(logits), _ptr(logits), _i64(_pitch(logits, cols)), _ptr(labels),
                                          _ptr(loss), _i64(rows), _i64(cols), _i64(ignored_index),
                                          stream if stream is not None else current_stream()))


def sce_sparse_bwd(logits, labels, grad_loss, dlogits, ignored_index, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    lv = _multi_level([logits, dlogits])
    if lv is not None:
        counts, (xs, ds) = lv
        check(lib().hk_sce_sparse_bwd_strided_rows(dtype_code(logits), _ptr(logits), _steps(xs), _ptr(labels),
                                                   _ptr(grad_loss), _ptr(dlogits), _steps(ds), _arr(counts),
                                                   _i64(cols), _i64(ignored_index),
                                                   stream if stream is not None else current_stream()))
        return
    check(lib().hk_sce_sparse_bwd_pitched(dtype_code(logits), _ptr(logits), _i64(_pitch(logits, cols)), _ptr(labels),
                                          _ptr(grad_loss), _ptr(dlogits), _i64(_pitch(dlogits, cols)), _i64(rows),
                                          _i64(cols), _i64(ignored_index),
                                          stream if stream is not None else current_stream()))


def sce_sparse_bwd_reduced(logits, labels, grad_output, scale, dlogits, ignored_index, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    check(lib().hk_sce_sparse_bwd_reduced(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(grad_output),
                                          ctypes.c_double(scale), _ptr(dlogits), _i64(rows), _i64(cols),
                                          _i64(ignored_index), stream if stream is not None else current_stream()))


def sce_dense_bwd_reduced(logits, labels, grad_output, scale, dlogits, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    check(lib().hk_sce_dense_bwd_reduced(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(grad_output),
                                         ctypes.c_double(scale), _ptr(dlogits), _i64(rows), _i64(cols),
                                         stream if stream is not None else current_stream()))


def sce_dense_fwd(logits, labels, loss, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    check(lib().hk_sce_dense_fwd(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(loss), _i64(rows), _i64(cols),
                                 stream if stream is not None else current_stream()))


def sce_dense_bwd(logits, labels, grad_loss, dlogits, stream=None):
    cols = logits.shape[-1]
    rows = logits.numel() // cols if logits.numel() else 0
    check(lib().hk_sce_dense_bwd(dtype_code(logits), _ptr(logits), _ptr(labels), _ptr(grad_loss), _ptr(dlogits),
                                 _i64(rows), _i64(cols), stream if stream is not None else current_stream()))


def nll_loss_fwd(pred, labels, loss, stream=None):
    cols = pred.shape[-1]
    rows = pred.numel() // cols if pred.numel() else 0
    check(lib().hk_nll_loss_fwd(dtype_code(pred), _ptr(pred), _ptr(labels), _ptr(loss), _i64(rows), _i64(cols),
                                stream if stream is not None else current_stream()))


def nll_loss_bwd(labels, grad_loss, out, stream=None):
    cols = out.shape[-1]
    rows = out.numel() // cols if out.numel() else 0
    check(lib().hk_nll_loss_bwd(dtype_code(out), _ptr(labels), _ptr(grad_loss), _ptr(out), _i64(rows), _i64(cols),
                                stream if stream is not None else current_stream()))


def reduce_workspace_bytes(dtype, shape, strides, axes):
    n = ctypes.c_size_t()
    check(lib().hk_reduce_workspace_bytes(ctypes.c_int(dtype), ctypes.c_int(len(shape)), _arr(shape), _arr(strides),
                                          ctypes.c_int(len(axes)), _arr(axes), ctypes.byref(n)))
    return n.value


def reduce(x, out, axes, op="sum", workspace=None, stream=None):
    """x may be any strided torch view; axes already wrapped to [0, ndim)."""
    shape, strides = list(x.shape), list(x.stride())
    if workspace is None:
        workspace = _workspace(reduce_workspace_bytes(dtype_code(x), shape, strides, axes), x.device)
    wsb = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib().hk_reduce(dtype_code(x), dtype_code(out), _ptr(x), _ptr(out), ctypes.c_int(len(shape)), _arr(shape),
                          _arr(strides), ctypes.c_int(len(axes)), _arr(axes),
                          ctypes.c_int(REDUCE_OPS[op]), _ptr(workspace),
                          ctypes.c_size_t(wsb), stream if stream is not None else current_stream()))
    return workspace


def copy_kernel(dst, src, stream=None):
    check(lib().hk_copy_kernel(_ptr(dst), _ptr(src), ctypes.c_size_t(src.numel() * src.element_size()),
                               stream if stream is not None else current_stream()))


def stream_probe(dsts, srcs, block_threads=256, vectors_per_thread=1, nt_loads=True, nt_stores=True,
                 workgroups_per_cu=0, stream=None):
    """Streaming yardstick: len(srcs) arrays read, len(dsts) arrays written, all of the first array's size."""
    ref = (list(srcs) + list(dsts))[0]
    nbytes = ref.numel() * ref.element_size()
    d = list(dsts) + [None, None]
    r = list(srcs) + [None, None]
    rc = bench_lib().hk_bench_stream_probe(_ptr(d[0]), _ptr(d[1]), _ptr(r[0]), _ptr(r[1]), ctypes.c_int(len(srcs)),
                                           ctypes.c_int(len(dsts)), ctypes.c_size_t(nbytes),
                                           ctypes.c_int(block_threads), ctypes.c_int(vectors_per_thread),
                                           ctypes.c_int(int(nt_loads)), ctypes.c_int(int(nt_stores)),
                                           ctypes.c_int(workgroups_per_cu),
                                           stream if stream is not None else current_stream())
    if rc != 0:
        raise HkError(rc, bench_lib().hk_bench_last_error().decode("utf-8", "replace"))


def ring_probe(dst, src0, src1, block_threads=512, depth=2, barrier=True, workgroups_per_cu=1, stream=None):
    """Pipelined persistent yardstick: two arrays read, one written, a ring of `depth` tiles in flight per thread."""
    nbytes = dst.numel() * dst.element_size()
    rc = bench_lib().hk_bench_ring_probe(_ptr(dst), _ptr(src0), _ptr(src1), ctypes.c_size_t(nbytes),
                                         ctypes.c_int(block_threads), ctypes.c_int(depth), ctypes.c_int(int(barrier)),
                                         ctypes.c_int(workgroups_per_cu),
                                         stream if stream is not None else current_stream())
    if rc != 0:
        raise HkError(rc, bench_lib().hk_bench_last_error().decode("utf-8", "replace"))


def memcpy_d2d(dst, src, stream=None):
    check(lib().hk_memcpy_d2d(_ptr(dst), _ptr(src), ctypes.c_size_t(src.numel() * src.element_size()),
                              stream if stream is not None else current_stream()))


def strided_copy(src, dst, stream=None):
    check(lib().hk_strided_copy(dtype_code(src), _ptr(src), _ptr(dst), ctypes.c_int(src.dim()), _arr(src.shape),
                                _arr(src.stride()), stream if stream is not None else current_stream()))


def strided_scatter(src, dst, stream=None):
    """Lays the dense array `src` over the view `dst` (same shape, any strides)."""
    check(lib().hk_strided_scatter(dtype_code(dst), _ptr(src), _ptr(dst), ctypes.c_int(dst.dim()), _arr(dst.shape),
                                   _arr(dst.stride()), stream if stream is not None else current_stream()))
