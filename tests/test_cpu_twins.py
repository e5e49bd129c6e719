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
    helpers.assert_close(tdx, edx, dtype, "dx")
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
