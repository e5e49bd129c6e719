"""The host ("Cpu") twins of the kernels, behind the same entry points and the same device dispatch as the accelerator
kernels (HT_DISPATCH_KERNEL_CPU_AND_CUDA): LayerNorm / LayerNormGradient, Softmax / SoftmaxGradient,
SoftmaxCrossEntropySparse / ...Gradient and Reduce on host arrays, compared with the oracle.  No GPU is needed."""
import importlib

import numpy as np
import pytest

import helpers
import oracle


@pytest.fixture(scope="module")
def ht():
    helpers.load_package()
    return importlib.import_module("hotspa-ae_amd.hetu_ops")


def _t(a, dtype):
    return helpers.to_torch(a, dtype, "cpu")


DTYPES = ["fp32", "bf16", "fp16", "fp64"]


def _draw(seed, shape, dtype, **kw):
    v = helpers.draw(seed, shape, dtype="fp32" if dtype == "fp64" else dtype, **kw)
    return v.astype(np.float64) if dtype == "fp64" else v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(7, 64), (33, 1000), (3, 4, 257), (128, 4096)])
def test_layer_norm_and_gradient(ht, dtype, shape):
    import torch
    cols = shape[-1]
    rows = int(np.prod(shape[:-1]))
    eps = 1e-5
    x = _draw(11, shape, dtype)
    gamma = _draw(12, (cols,), dtype, dist="uniform", a=0.5, b=1.5)
    beta = _draw(13, (cols,), dtype, dist="normal", a=0.0, b=0.1)
    dy = _draw(14, shape, dtype)
    ey, emean, evar, _ = oracle.layernorm_fwd(x.reshape(rows, cols), gamma, beta, eps)
    tx, tg, tb, tdy = (_t(v, dtype) for v in (x, gamma, beta, dy))
    ty = torch.empty_like(tx)
    stat_shape = list(shape[:-1]) + [1]
    tmean = torch.empty(stat_shape, dtype=tx.dtype)
    tvar = torch.empty(stat_shape, dtype=tx.dtype)
    ht.layer_norm(tx, tg, tb, tmean, tvar, ty, 1, eps)
    helpers.assert_close(ty.reshape(rows, cols), ey, dtype, "y")
    helpers.assert_close(tmean.reshape(rows), emean, dtype, "mean", scale=1.0)
    helpers.assert_close(tvar.reshape(rows), evar, dtype, "var")
    # gradient from the stored (rounded) statistics, as the accelerator kernel is tested
    mean_s = helpers.to_numpy(tmean).reshape(rows).astype(np.float64)
    var_s = helpers.to_numpy(tvar).reshape(rows).astype(np.float64)
    rstd = 1.0 / np.sqrt(var_s + eps)
    edx, edg, edb = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), gamma, mean_s, rstd, eps)
    tdx, tdg, tdb = torch.empty_like(tx), torch.empty_like(tg), torch.empty_like(tg)
    ht.layer_norm_gradient(tdy, tx, tg, tdx, tdg, tdb, tmean, tvar, 1, eps)
    helpers.assert_close(tdx.reshape(rows, cols), edx, dtype, "dx")
    helpers.assert_close(tdg, edg, dtype, "dgamma", scale=float(np.sqrt(rows)))
    helpers.assert_close(tdb, edb, dtype, "dbeta", scale=float(np.sqrt(rows)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,dim", [((5, 100), -1), ((4, 6, 50), 1), ((3, 7, 9), 0), ((64, 2048), 1)])
def test_softmax_and_gradient(ht, dtype, shape, dim):
    import torch
    x = _draw(21, shape, dtype, b=3.0)
    dy = _draw(22, shape, dtype)
    ey = oracle.softmax_fwd(x, dim)
    tx = _t(x, dtype)
    ty = torch.empty_like(tx)
    ht.softmax(tx, ty, dim)
    helpers.assert_close(ty, ey, dtype, "sm_y")
    y = helpers.to_numpy(ty).astype(np.float64)
    if dtype == "fp64":   # the oracle's C entry takes fp32-valued inputs; this y is not: the closed form in numpy
        edx = y * (dy - np.sum(dy * y, axis=dim, keepdims=True))
    else:
        edx = oracle.softmax_bwd(y, dy, dim)
    tdx = torch.empty_like(tx)
    ht.softmax_gradient(ty, _t(dy, dtype), tdx, dim)
    helpers.assert_close(tdx, edx, dtype, "dx", ordinary_rtol=helpers.SOFTMAX_GRADIENT_ORDINARY_RTOL)
    # a transposed input is read through its strides
    if len(shape) == 2:
        txt = _t(np.ascontiguousarray(x.T), dtype).t()
        ty2 = torch.empty_like(ty)
        ht.softmax(txt, ty2, dim)
        assert torch.equal(ty2, ty)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(9, 17), (4, 8, 1000), (256, 32000)])
def test_sparse_cross_entropy_and_gradient(ht, dtype, shape):
    import torch
    if dtype != "fp32" and shape[-1] == 32000:
        pytest.skip("the large case once")
    cols = shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = _draw(31, shape, dtype, b=2.0)
    g = helpers.rng(32)
    labels = g.integers(0, cols, size=shape[:-1]).astype(np.int64)
    labels.reshape(-1)[::5] = -100
    gl = _draw(33, shape[:-1], dtype)
    eloss = oracle.sce_sparse_fwd(x.reshape(rows, cols), labels.reshape(rows), -100)
    edx = oracle.sce_sparse_bwd(x.reshape(rows, cols), labels.reshape(rows), gl.reshape(rows), -100)
    tx, tl, tgl = _t(x, dtype), torch.from_numpy(labels), _t(gl, dtype)
    tloss = torch.empty(shape[:-1], dtype=tx.dtype)
    ht.softmax_cross_entropy_sparse(tx, tl, tloss, -100)
    helpers.assert_close(tloss.reshape(rows), eloss, dtype, "loss")
    tdx = torch.empty_like(tx)
    ht.softmax_cross_entropy_sparse_gradient(tx, tl, tgl, tdx, -100)
    helpers.assert_close(tdx.reshape(rows, cols), edx, dtype, "dlogits")
    ign = labels.reshape(rows) == -100
    assert np.all(helpers.to_numpy(tloss).reshape(rows)[ign] == 0)
    assert np.all(helpers.to_numpy(tdx).reshape(rows, cols)[ign] == 0)
    # a label outside the classes that is not the ignored one: NaN, not an out-of-bounds read
    bad = labels.copy()
    bad.reshape(-1)[1] = cols + 3
    ht.softmax_cross_entropy_sparse(tx, torch.from_numpy(bad), tloss, -100)
    assert np.isnan(helpers.to_numpy(tloss).reshape(rows)[1])


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp64"])
@pytest.mark.parametrize("op", ["sum", "mean", "max", "min", "prod"])
def test_reduce_every_axis_subset(ht, dtype, op):
    import itertools
    import torch
    shape = (3, 4, 5, 6)
    x = _draw(41, shape, dtype, dist="uniform", a=0.5, b=1.5) if op == "prod" else _draw(41, shape, dtype)
    tx = _t(x, dtype)
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            want = oracle.reduce(x, list(axes), op)
            out = torch.empty([s for i, s in enumerate(shape) if i not in axes] or [1], dtype=tx.dtype)
            ht.reduce(tx, out, list(axes), op)
            # the mean multiplies the sum by float(1 / count), a single-precision factor, for every type (as the
            # accelerator kernel and ReduceMean.cu:9-22 do): 6e-8 relative for a count that is no power of two
            helpers.assert_close(out.reshape(np.asarray(want).shape), want, dtype, "%s %s" % (op, axes),
                                 scale=float(np.abs(want).max()) if op in ("sum", "mean") else None,
                                 rtol=1e-7 if (dtype == "fp64" and op == "mean") else None)
    # a permuted view is read in place
    xt = tx.permute(2, 0, 3, 1)
    want = oracle.reduce(np.ascontiguousarray(np.transpose(x, (2, 0, 3, 1))), [1, 2], op)
    out = torch.empty(want.shape, dtype=tx.dtype)
    ht.reduce(xt, out, [1, 2], op)
    helpers.assert_close(out, want, dtype, "%s permuted" % op, scale=float(np.abs(want).max()),
                         rtol=1e-7 if (dtype == "fp64" and op == "mean") else None)


def test_reduce_integers_and_large(ht):
    import torch
    g = helpers.rng(51)
    xi = g.integers(-50, 50, size=(300, 257)).astype(np.int64)
    for axes in ([0], [1], [0, 1]):
        out = torch.empty([s for i, s in enumerate(xi.shape) if i not in axes] or [1], dtype=torch.int64)
        ht.reduce(torch.from_numpy(xi), out, axes, "sum")
        assert np.array_equal(out.numpy().reshape(-1), xi.sum(axis=tuple(axes)).reshape(-1))
    x = helpers.draw(52, (4096, 4096), dtype="fp32")
    for axes in ([0], [1]):
        out = torch.empty(4096)
        ht.reduce(torch.from_numpy(x), out, axes, "mean")
        want = x.astype(np.float64).mean(axis=axes[0])
        helpers.assert_close(out, want, "fp32", "mean %s" % axes, scale=float(np.abs(want).max()))


def test_ndarray_statics_dispatch_on_the_device(ht):
    """NDArray::softmax / reduce / layernorm / sceloss on host arrays reach the host twins through
    HT_DISPATCH_KERNEL_CPU_AND_CUDA."""
    import torch
    x = helpers.draw(61, (12, 40), dtype="fp32")
    tx = torch.from_numpy(x)
    out = torch.empty_like(tx)
    ht.ndarray_softmax(tx, -1, out)
    helpers.assert_close(out, oracle.softmax_fwd(x), "fp32", "sm_y")
    red = torch.empty(40)
    ht.ndarray_reduce(tx, "mean", [0], False, red)
    helpers.assert_close(red, oracle.reduce(x, [0], "mean"), "fp32", "mean", scale=1.0)
    labels = torch.from_numpy(helpers.rng(62).integers(0, 40, size=(12,)).astype(np.int64))
    loss = torch.empty(1)
    ht.ndarray_sceloss(tx, labels, loss, "mean", -100)
    want = oracle.sce_sparse_fwd(x, labels.numpy(), -100).mean()
    assert abs(float(loss) - want) <= 1e-5 * abs(want)
    g = torch.ones(40)
    b = torch.zeros(40)
    y = torch.empty_like(tx)
    ht.ndarray_layernorm(tx, g, b, 1, 1e-5, False, y)
    helpers.assert_close(y, oracle.layernorm_fwd(x, np.ones(40, np.float32), np.zeros(40, np.float32), 1e-5)[0],
                         "fp32", "y")


def test_host_and_accelerator_arrays_do_not_mix(ht):
    import torch
    x = torch.zeros(4, 8)
    with pytest.raises(ht.HetuError):
        ht.softmax(x, torch.empty(4, 9), -1)          # shape mismatch is caught before any loop runs
    with pytest.raises(ht.HetuError):
        ht.reduce(x, torch.empty(5), [0], "sum")


# ---- the neighbours of the row-wise kernels: element-wise family, dense / NLL losses, broadcasts, norms ------------
def _round(a, dtype):
    return a if dtype == "fp64" else oracle.round_to(np.asarray(a, np.float32), dtype).astype(np.float64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shapes", [((6, 50), (6, 50)), ((6, 50), (50,)), ((6, 1), (1, 50)), ((4, 1, 7), (3, 1)),
                                    ((), (5,)), ((300, 400), (300, 1))])
def test_binary_broadcasting(ht, dtype, shapes):
    import torch
    sa, sb = shapes
    a = _draw(71, sa, dtype)
    b = _draw(72, sb, dtype, dist="uniform", a=0.5, b=2.0)
    for op, f in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        want = f(a.astype(np.float64), b.astype(np.float64))
        out = torch.empty(want.shape, dtype=_t(a, dtype).dtype)
        ht.binary(op, _t(a, dtype), _t(b, dtype), out)
        if dtype == "fp64":
            assert np.array_equal(helpers.to_numpy(out), want)
        elif dtype == "fp32":   # one IEEE operation: the float32 result itself
            assert np.array_equal(helpers.to_numpy(out), f(a, b))
        else:   # computed in float32, rounded once
            assert np.array_equal(helpers.to_numpy(out).astype(np.float64), _round(f(a, b), dtype))


def test_binary_reads_operands_through_their_strides(ht):
    import torch
    a = torch.arange(24, dtype=torch.float32).reshape(4, 6)
    b = torch.arange(24, dtype=torch.float32).reshape(6, 4).t()   # transposed view
    out = torch.empty(4, 6)
    ht.binary("sub", a, b, out)
    assert torch.equal(out, a - b)
    o2 = torch.empty(4, 3)                                         # column slices
    ht.binary("mul", a[:, ::2], b[:, 1::2], o2)
    assert torch.equal(o2, a[:, ::2] * b[:, 1::2])
    with pytest.raises(ht.HetuError):
        ht.binary("add", a, torch.zeros(5), out)


@pytest.mark.parametrize("tname", ["uint8", "int8", "int16", "int32", "int64"])
def test_integer_arithmetic_wraps(ht, tname):
    import torch
    td = getattr(torch, tname)
    nd = np.dtype(tname)
    info = np.iinfo(nd)
    g = helpers.rng(73)
    a = g.integers(info.min, info.max, size=(5, 33), dtype=nd, endpoint=True)
    b = g.integers(info.min, info.max, size=(33,), dtype=nd, endpoint=True)
    b[::7] = 0
    if info.min < 0:
        a[0, 1], b[1] = info.min, -1   # the quotient that does not fit
    ta, tb = torch.from_numpy(a), torch.from_numpy(b)
    out = torch.empty(5, 33, dtype=td)
    with np.errstate(over="ignore"):
        for op, f in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply)):
            ht.binary(op, ta, tb, out)
            assert np.array_equal(out.numpy(), f(a, b)), op
    ht.binary("div", ta, tb, out)
    wide_a, wide_b = a.astype(object), np.broadcast_to(b, a.shape).astype(object)
    want = np.zeros(a.shape, dtype=object)
    nz = wide_b != 0
    # C division truncates towards zero
    q = np.vectorize(lambda x, y: abs(x) // abs(y) * (1 if (x >= 0) == (y >= 0) else -1), otypes=[object])(
        wide_a[nz], wide_b[nz])
    want[nz] = q
    span = int(info.max) - int(info.min) + 1
    want = np.vectorize(lambda v: (int(v) - int(info.min)) % span + int(info.min), otypes=[object])(want).astype(nd)
    assert np.array_equal(out.numpy(), want)
    ht.unary("neg", ta, out)
    with np.errstate(over="ignore"):
        assert np.array_equal(out.numpy(), np.negative(a))
    ht.binary_const("sub", ta, 3.0, out)
    with np.errstate(over="ignore"):
        assert np.array_equal(out.numpy(), np.subtract(nd.type(3), a))
    with pytest.raises(ht.HetuError):
        ht.unary("exp", ta, out)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unary_and_constants(ht, dtype):
    import torch
    x = _draw(74, (37, 129), dtype, dist="uniform", a=0.25, b=4.0)
    tx = _t(x, dtype)
    out = torch.empty_like(tx)
    for op, f in (("exp", np.exp), ("log", np.log), ("sqrt", np.sqrt), ("neg", np.negative)):
        ht.unary(op, tx, out)
        helpers.assert_close(out, f(x.astype(np.float64)), dtype, op)
    c = 1.7
    cr = float(np.asarray(_round(np.float64(c), dtype)).reshape(-1)[0])   # the constant is rounded to the array's type first
    xd = x.astype(np.float64)
    for op, want in (("add", cr + xd), ("sub", cr - xd), ("mul", cr * xd), ("div", cr / xd)):
        ht.binary_const(op, tx, c, out)
        helpers.assert_close(out, want, dtype, "const " + op)
    with pytest.raises(ht.HetuError, match="Divided by 0"):
        ht.binary_const("div", tx, 0.0, out)
    # special values pass through as IEEE says
    s = torch.tensor([0.0, -1.0, float("inf"), float("nan")])
    o = torch.empty(4)
    ht.unary("log", s, o)
    assert o[0] == -float("inf") and torch.isnan(o[1]) and o[2] == float("inf") and torch.isnan(o[3])
    ht.unary("sqrt", s, o)
    assert o[0] == 0 and torch.isnan(o[1]) and o[2] == float("inf") and torch.isnan(o[3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(9, 17), (4, 8, 1000)])
def test_dense_cross_entropy_and_gradient(ht, dtype, shape):
    import torch
    cols = shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = _draw(75, shape, dtype, b=2.0)
    lab = helpers.rng(76).random(shape, dtype=np.float32)
    lab = lab / lab.sum(axis=-1, keepdims=True)
    lab = lab.astype(np.float64) if dtype == "fp64" else oracle.round_to(lab, dtype)
    gl = _draw(77, shape[:-1], dtype)
    tx, tl, tgl = _t(x, dtype), _t(lab, dtype), _t(gl, dtype)
    loss = torch.empty(shape[:-1], dtype=tx.dtype)
    ht.softmax_cross_entropy(tx, tl, loss)
    helpers.assert_close(loss.reshape(rows), oracle.sce_dense_fwd(x.reshape(rows, cols), lab.reshape(rows, cols)),
                         dtype, "loss")
    dx = torch.empty_like(tx)
    ht.softmax_cross_entropy_gradient(tx, tl, tgl, dx)
    helpers.assert_close(dx.reshape(rows, cols),
                         oracle.sce_dense_bwd(x.reshape(rows, cols), lab.reshape(rows, cols), gl.reshape(rows)),
                         dtype, "dlogits")


@pytest.mark.parametrize("dtype", DTYPES)
def test_nll_loss_and_gradient(ht, dtype):
    import torch
    rows, cols = 41, 23
    pred = _draw(78, (rows, cols), dtype)
    labels = helpers.rng(79).integers(0, cols, size=(rows,)).astype(np.int64)
    labels[3], labels[7] = -1, cols   # outside the classes: loss 0, gradient row 0
    gl = _draw(80, (rows,), dtype)
    tp, tl, tg = _t(pred, dtype), torch.from_numpy(labels), _t(gl, dtype)
    loss = torch.empty(rows, dtype=tp.dtype)
    ht.nll_loss(tp, tl, loss)
    assert np.array_equal(helpers.to_numpy(loss).astype(np.float64), oracle.nll_loss_fwd(pred, labels))
    dx = torch.full((rows, cols), 7.0, dtype=tp.dtype)
    ht.nll_loss_gradient(tp, tl, tg, dx)
    helpers.assert_close(dx, oracle.nll_loss_bwd(labels, gl, cols), dtype, "dpred")
    assert np.all(helpers.to_numpy(dx)[[3, 7]] == 0)


@pytest.mark.parametrize("case", [((5,), (3, 5), ()), ((3, 1), (3, 5), ()), ((3, 5), (2, 3, 4, 5), (0, 2)),
                                  ((4,), (4, 6), (1,)), ((), (2, 3), ()), ((1, 6), (7, 6), ()),
                                  ((200,), (300, 200), ())])
@pytest.mark.parametrize("dtype", ["fp32", "bf16", "int32"])
def test_broadcast_shape(ht, dtype, case):
    import torch
    in_shape, out_shape, add_axes = case
    if dtype == "int32":
        x = helpers.rng(81).integers(-1000, 1000, size=in_shape, dtype=np.int32)
        tx = torch.from_numpy(np.asarray(x))
    else:
        x = _draw(81, in_shape, dtype)
        tx = _t(x, dtype)
    out = torch.empty(out_shape, dtype=tx.dtype)
    ht.broadcast_shape(tx, out, add_axes)
    assert np.array_equal(helpers.to_numpy(out), oracle.broadcast_shape(x, out_shape, add_axes).astype(x.dtype))
    ht.broadcast_shape(tx, out, add_axes, const_value=0.5 if dtype != "int32" else 3)
    want = oracle.broadcast_shape(x, out_shape, add_axes, const_value=0.5 if dtype != "int32" else 3)
    if dtype == "int32":
        assert np.array_equal(out.numpy(), want.astype(np.int32))
    else:
        helpers.assert_close(out, want, dtype, "broadcast * c")
    with pytest.raises(ht.HetuError):
        ht.broadcast_shape(torch.zeros(4), torch.empty(3, 5), ())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("p", [1, 2, 3])
@pytest.mark.parametrize("shape,dim", [((6, 40), 1), ((6, 40), 0), ((3, 5, 7), 1), ((2, 3000), -1)])
def test_norm_and_gradient(ht, dtype, p, shape, dim):
    import torch
    x = _draw(82, shape, dtype)
    x.reshape(-1)[::11] = 0
    if len(shape) == 3:
        x[1, :, 2] = 0   # a zero norm: its gradient is 0, not NaN
    kept = tuple(s for i, s in enumerate(shape) if i != dim % len(shape))
    g = _draw(83, kept, dtype)
    tx = _t(x, dtype)
    n = torch.empty(kept, dtype=tx.dtype)
    ht.norm(tx, n, dim, p)
    helpers.assert_close(n, oracle.norm_p_fwd(x, dim, p), dtype, "norm")
    dx = torch.empty_like(tx)
    ht.norm_gradient(tx, n, _t(g, dtype), dx, dim, p)
    stored = helpers.to_numpy(n).astype(np.float64)
    helpers.assert_close(dx, oracle.norm_p_bwd(x, stored, g, dim % len(shape), p), dtype, "dx")
    with pytest.raises(ht.HetuError):
        ht.norm(tx, n, dim, 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3, 5, 7), (1, 4, 32, 32)])
def test_instance_norm_and_gradient(ht, dtype, shape):
    import torch
    rows, cols = shape[0] * shape[1], shape[2] * shape[3]
    eps = 1e-5
    x = _draw(84, shape, dtype, a=0.5)
    dy = _draw(85, shape, dtype)
    ones, zeros = np.ones(cols, np.float32), np.zeros(cols, np.float32)
    ey, emean, evar, _ = oracle.layernorm_fwd(x.reshape(rows, cols), ones, zeros, eps)
    tx = _t(x, dtype)
    y = torch.empty_like(tx)
    mean = torch.empty(shape[0], shape[1], 1, 1, dtype=tx.dtype)
    var = torch.empty_like(mean)
    ht.instance_norm(tx, mean, var, y, eps)
    helpers.assert_close(y.reshape(rows, cols), ey, dtype, "y")
    helpers.assert_close(mean.reshape(rows), emean, dtype, "mean", scale=1.0)
    helpers.assert_close(var.reshape(rows), evar, dtype, "var")
    ms = helpers.to_numpy(mean).reshape(rows).astype(np.float64)
    vs = helpers.to_numpy(var).reshape(rows).astype(np.float64)
    edx, _, _ = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), ones, ms, 1 / np.sqrt(vs + eps),
                                     eps)
    dx = torch.empty_like(tx)
    ht.instance_norm_gradient(_t(dy, dtype), tx, dx, mean, var, eps)
    helpers.assert_close(dx.reshape(rows, cols), edx, dtype, "dx")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 3, 5, 7), (8, 16), (2, 5, 33), (1, 2, 1, 1)])
def test_batch_norm_and_gradient(ht, dtype, shape):
    import torch
    C = shape[1]
    pdt = "fp64" if dtype == "fp64" else "fp32"   # parameters and statistics: float32 for 16-bit data
    eps, momentum = 1e-5, 0.1
    x = _draw(86, shape, dtype, a=0.3)
    dy = _draw(87, shape, dtype)
    scale = _draw(88, (C,), pdt, dist="uniform", a=0.5, b=1.5)
    bias = _draw(89, (C,), pdt, b=0.1)
    rm0 = _draw(90, (C,), pdt)
    rv0 = _draw(91, (C,), pdt, dist="uniform", a=0.5, b=1.5)
    ey, erm, erv, emean, einv = oracle.batch_norm_fwd(x, scale, bias, rm0, rv0, momentum, eps)
    tx, ts, tb = _t(x, dtype), _t(scale, pdt), _t(bias, pdt)
    rm, rv = _t(rm0, pdt).clone(), _t(rv0, pdt).clone()
    sm, sv = torch.empty_like(rm), torch.empty_like(rm)
    y = torch.empty_like(tx)
    ht.batch_norm(tx, ts, tb, y, momentum, eps, rm, rv, sm, sv)
    one_value = x.size // C == 1   # var = 0: y = bias, inverse deviation 1 / sqrt(eps)
    helpers.assert_close(y, ey, dtype, "y", scale=1.0 if one_value else None)
    helpers.assert_close(sm, emean, pdt, "save_mean", scale=1.0)
    helpers.assert_close(sv, einv, pdt, "save_invstd")
    helpers.assert_close(rm, erm, pdt, "running_mean", scale=1.0)
    helpers.assert_close(rv, erv, pdt, "running_var")
    edx, eds, edb = oracle.batch_norm_bwd(dy, x, scale, helpers.to_numpy(sm), helpers.to_numpy(sv))
    dx, ds, db = torch.empty_like(tx), torch.empty_like(rm), torch.empty_like(rm)
    ht.batch_norm_gradient(_t(dy, dtype), tx, ts, dx, ds, db, eps, sm, sv)
    m = x.size // C
    if not one_value:
        helpers.assert_close(dx, edx, dtype, "dx")
    helpers.assert_close(ds, eds, pdt, "dscale", scale=float(np.sqrt(m)))
    helpers.assert_close(db, edb, pdt, "dbias", scale=float(np.sqrt(m)))
    with pytest.raises(ht.HetuError):
        ht.batch_norm(tx, ts.to(torch.float16), tb, y, momentum, eps, rm, rv, sm, sv)


def test_ndarray_arithmetic_statics_on_host_arrays(ht):
    """NDArray::add / sub / mul / div / exp / neg / norm and the dense sceloss on host arrays reach the host twins."""
    import torch
    a = torch.from_numpy(helpers.draw(92, (6, 10), dtype="fp32"))
    b = torch.from_numpy(helpers.draw(93, (10,), dtype="fp32", dist="uniform", a=0.5, b=2.0))
    out = torch.empty(6, 10)
    for op, f in (("add", torch.add), ("sub", torch.sub), ("mul", torch.mul), ("div", torch.div)):
        ht.ndarray_binary(op, a, b, out)
        assert torch.equal(out, f(a, b)), op
    ht.ndarray_unary("neg", a, out)
    assert torch.equal(out, -a)
    n = torch.empty(6)
    ht.ndarray_norm(a, 2, 1, False, n)
    helpers.assert_close(n, oracle.norm_p_fwd(a.numpy(), 1, 2), "fp32", "norm")
    lab = torch.softmax(torch.from_numpy(helpers.draw(94, (6, 10), dtype="fp32")), dim=1)
    loss = torch.empty(1)
    ht.ndarray_sceloss(a, lab, loss, "sum")
    want = oracle.sce_dense_fwd(a.numpy(), lab.numpy()).sum()
    assert abs(float(loss) - want) <= 1e-5 * abs(want)


def test_host_calls_on_a_stream_run_in_order_and_report_failures_at_sync(ht):
    """Host streams 1..15 are task queues with a worker thread each (the blocking stream 0 runs in the caller).  With
    the C face switched to asynchronous host calls, a chain of dependent kernels on one stream gives the bits of the
    same chain run call by call, and the first failure of a task comes out of the stream's sync."""
    import torch
    x = _t(_draw(71, (256, 384), "fp32"), "fp32")

    def chain(stream):
        y, e = torch.zeros_like(x), torch.zeros_like(x)
        s = torch.zeros((256,), dtype=x.dtype)
        ht.softmax(x, y, 1, stream=stream)
        ht.unary("exp", y, e, stream=stream)
        ht.reduce(e, s, [1], "sum", stream=stream)
        return y, e, s

    want = chain(0)
    was = ht.set_host_async(True)
    try:
        assert was is False
        got = chain(7)
        ht.host_stream_sync(7)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        # argument checks still fail the call itself
        with pytest.raises(ht.HetuError):
            ht.softmax(x, torch.zeros((256, 385)), 1, stream=7)
        ht.host_stream_sync(7)
    finally:
        ht.set_host_async(False)
        ht.synchronize_all()
    # default mode: the call has finished when it returns, whatever the stream
    y = torch.zeros_like(x)
    ht.softmax(x, y, 1, stream=9)
    assert torch.equal(y, want[0])


@pytest.mark.parametrize("level", [0, 1])
def test_every_instruction_set_variant_of_the_host_loops(level):
    """The inner loops of the host kernels are compiled for baseline x86-64, AVX2 + FMA and AVX-512 and chosen once
    per process; the rest of this file runs the best the processor has.  The lower levels are forced through
    HETU_HOST_ISA in a process of their own, on the tests that cover every loop helper (sums, maxima, element-wise
    passes with and without exp)."""
    import os
    import subprocess
    import sys
    env = dict(os.environ, HETU_HOST_ISA=str(level))
    picked = ("test_layer_norm_and_gradient or test_softmax_and_gradient or test_sparse_cross_entropy_and_gradient "
              "or test_reduce_every_axis_subset or test_unary_and_constants or test_batch_norm_and_gradient "
              "or test_special_values_go_through_the_vector_loops")
    run = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-k", picked,
                          "-p", "no:cacheprovider"], env=env, cwd=helpers.ROOT, capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-3000:] + run.stderr[-2000:]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_special_values_go_through_the_vector_loops(ht, dtype):
    """-inf elements, a row of -inf only, +inf, NaN, a large common offset and an overflowing exponent: the
    branch-free exp and the lane-wise maxima give what the scalar library calls give."""
    import torch
    inf, nan = float("inf"), float("nan")
    dt = torch.float32 if dtype == "fp32" else torch.bfloat16
    x = torch.from_numpy(_draw(91, (6, 200), "fp32")).to(dt)
    x[0, 3] = -inf
    x[1, :] = -inf
    x[2, 5] = inf
    x[3, 7] = nan
    x[4, :] += 1e4
    x[5, 0] = 200.0
    y = torch.empty_like(x)
    ht.softmax(x, y, 1)
    ref = torch.softmax(x.double(), 1)
    assert torch.equal(torch.isnan(y), torch.isnan(ref))
    tol = 1e-5 if dtype == "fp32" else 1e-2
    assert torch.allclose(torch.nan_to_num(y.double()), torch.nan_to_num(ref), rtol=tol, atol=1e-7)
    e = torch.empty_like(x)
    ht.unary("exp", x, e)
    re = torch.exp(x.double()).to(dt)          # overflow where the type overflows
    assert torch.equal(torch.isnan(e), torch.isnan(re)) and torch.equal(torch.isinf(e), torch.isinf(re))
    fin = torch.isfinite(re)
    assert torch.allclose(e[fin].double(), re[fin].double(), rtol=tol, atol=0)
    assert float(e[1].abs().max()) == 0.0      # exp(-inf) is exactly 0
