"""GPU parity of the C++ operator layer (hetu::impl::<Kernel>Cuda entry points and
the NDArray statics) against the oracle, called through include/hetu_ops_c.h with
torch tensors as borrowed arrays.  The layer runs on its own HIP streams, so each
test drains torch's stream before the call and the layer's stream after it."""
import importlib

import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(hk):
    return importlib.import_module("hotspa-ae_amd.hetu_ops")


def _sync_in():
    import torch
    torch.cuda.synchronize()


def _dev(vals, dtype, cuda):
    return [helpers.to_torch(v, dtype, cuda) for v in vals]


def _norm_inputs(shape, cols, dtype, seed):
    x = helpers.draw(seed, shape, dtype=dtype)
    gamma = helpers.draw(seed + 1, (cols,), "uniform", 0.5, 1.5, dtype)
    beta = helpers.draw(seed + 2, (cols,), "normal", 0.0, 0.1, dtype)
    dy = helpers.draw(seed + 3, shape, dtype=dtype)
    return x, gamma, beta, dy


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape,reduce_dims", [((6, 5, 256), 1), ((3, 4, 16, 64), 2), ((33, 1000), 1)])
def test_layer_norm_and_gradient(ops, cuda, dtype, shape, reduce_dims):
    import torch
    cols = int(np.prod(shape[len(shape) - reduce_dims:]))
    rows = int(np.prod(shape)) // cols
    eps = 1e-5
    x, gamma, beta, dy = _norm_inputs(shape, cols, dtype, 11 + cols)
    ey, emean, evar, erstd = oracle.layernorm_fwd(x.reshape(rows, cols), gamma, beta, eps)
    tx, tg, tb, tdy = _dev((x, gamma, beta, dy), dtype, cuda)
    tg = tg.reshape(shape[len(shape) - reduce_dims:])
    tb = tb.reshape(shape[len(shape) - reduce_dims:])
    stat_shape = tuple(shape[:len(shape) - reduce_dims]) + (1,) * reduce_dims
    ty = torch.empty_like(tx)
    tmean = torch.empty(stat_shape, dtype=tx.dtype, device=cuda)
    tvar = torch.empty(stat_shape, dtype=tx.dtype, device=cuda)
    _sync_in()
    ops.layer_norm(tx, tg, tb, tmean, tvar, ty, reduce_dims, eps)
    ops.stream_sync()
    helpers.assert_close(ty, ey.reshape(shape), dtype, "y")
    helpers.assert_close(tvar.reshape(rows), evar, dtype, "var")
    # gradient from the statistics the forward stored (rounded to the data dtype, as the reference keeps them)
    mean_r = helpers.to_numpy(tmean).reshape(rows).astype(np.float64)
    var_r = helpers.to_numpy(tvar).reshape(rows).astype(np.float64)
    rstd_r = 1.0 / np.sqrt(var_r + eps)
    edx, edg, edb = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), gamma,
                                         mean_r.astype(np.float32), rstd_r.astype(np.float32))
    tdx = torch.empty_like(tx)
    tdg = torch.empty_like(tg)
    tdb = torch.empty_like(tg)
    _sync_in()
    ops.layer_norm_gradient(tdy, tx, tg, tdx, tdg, tdb, tmean, tvar, reduce_dims, eps)
    ops.stream_sync()
    helpers.assert_close(tdx, edx.reshape(shape), dtype, "dx")
    helpers.assert_close(tdg.reshape(cols), edg, dtype, "dscale")
    helpers.assert_close(tdb.reshape(cols), edb, dtype, "dbias")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("inplace", [False, True])
def test_fused_layer_norm_and_gradient(ops, cuda, dtype, inplace):
    import torch
    shape, cols = (4, 9, 512), 512
    rows = 36
    eps = 1e-5
    x, gamma, beta, dy = _norm_inputs(shape, cols, dtype, 77)
    ey, emean, _, erstd = oracle.layernorm_fwd(x.reshape(rows, cols), gamma, beta, eps)
    tx, tg, tb, tdy = _dev((x, gamma, beta, dy), dtype, cuda)
    ty = torch.empty_like(tx)
    tmean = torch.empty((4, 9, 1), dtype=torch.float32, device=cuda)
    trstd = torch.empty((4, 9, 1), dtype=torch.float32, device=cuda)
    _sync_in()
    ops.fused_layer_norm(tx, tg, tb, tmean, trstd, ty, 1, eps)
    ops.stream_sync()
    helpers.assert_close(ty, ey.reshape(shape), dtype, "y")
    helpers.assert_close(trstd.reshape(rows), erstd, "fp32", "rstd")
    mean32 = helpers.to_numpy(tmean).reshape(rows)
    rstd32 = helpers.to_numpy(trstd).reshape(rows)
    tdx, tdg, tdb = torch.empty_like(tx), torch.empty_like(tg), torch.empty_like(tg)
    if inplace:
        y_stored = helpers.to_numpy(ty).reshape(rows, cols)
        edx, edg, edb = oracle.layernorm_bwd_memeff(dy.reshape(rows, cols), y_stored, gamma, beta, rstd32, eps)
        _sync_in()
        ops.fused_layer_norm_gradient(tdy, ty, tg, tb, tdx, tdg, tdb, tmean, trstd, 1, eps, True)
    else:
        edx, edg, edb = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), gamma, mean32, rstd32,
                                             eps, clamp_gamma=True)
        _sync_in()
        ops.fused_layer_norm_gradient(tdy, tx, tg, tb, tdx, tdg, tdb, tmean, trstd, 1, eps, False)
    ops.stream_sync()
    helpers.assert_close(tdx, edx.reshape(shape), dtype, "dx")
    helpers.assert_close(tdg, edg, dtype, "dscale")
    helpers.assert_close(tdb, edb, dtype, "dbias")
    # statistics must be float32 for the fused variant
    with pytest.raises(ops.AssertionError_, match="float32"):
        ops.fused_layer_norm(tx, tg, tb, tmean.to(tx.dtype) if dtype != "fp32" else tmean.double(), trstd, ty, 1, eps)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("is_rms", [True, False])
@pytest.mark.parametrize("with_residual", [False, True])
def test_dropout_add_ln(ops, cuda, dtype, is_rms, with_residual):
    import torch
    rows, cols = 48, 4096
    eps = 1e-6
    x0, gamma, beta, dz = _norm_inputs((rows, cols), cols, dtype, 300 + int(is_rms))
    res = helpers.draw(305, (rows, cols), dtype=dtype) if with_residual else None
    ez, ex, emu, ers = oracle.dropout_add_ln_fwd(x0, res, gamma, None if is_rms else beta, eps, is_rms)
    tx0, tg, tb, tdz = _dev((x0, gamma, beta, dz), dtype, cuda)
    tres = helpers.to_torch(res, dtype, cuda) if with_residual else None
    tz = torch.empty_like(tx0)
    tx = torch.empty_like(tx0) if with_residual else None
    tmu = torch.empty(rows, dtype=torch.float32, device=cuda)
    trs = torch.empty(rows, dtype=torch.float32, device=cuda)
    _sync_in()
    ops.dropout_add_ln_fwd(tx0, tres, tg, None if is_rms else tb, tz, tx, tmu, trs, eps, is_rms)
    ops.stream_sync()
    helpers.assert_close(tz, ez, dtype, "z")
    helpers.assert_close(trs, ers, "fp32", "rsigma")
    if with_residual:
        helpers.assert_close(tx, ex, dtype, "x")
    x_saved = helpers.to_numpy(tx) if with_residual else x0
    mu32, rs32 = helpers.to_numpy(tmu), helpers.to_numpy(trs)
    edx0, edg, edb = oracle.dropout_add_ln_bwd(dz, None, x_saved, mu32, rs32, gamma, is_rms)
    tdx0 = torch.empty_like(tx0)
    tdres = torch.empty_like(tx0) if with_residual else None
    tdg, tdb = torch.empty_like(tg), torch.empty_like(tg)
    _sync_in()
    ops.dropout_add_ln_bwd(tdz, None, tx if with_residual else tx0, tmu, trs, tg, tdx0, tdres, tdg, tdb,
                           with_residual, is_rms)
    ops.stream_sync()
    helpers.assert_close(tdx0, edx0, dtype, "dx0")
    helpers.assert_close(tdg, edg, dtype, "dgamma")
    helpers.assert_close(tdb, edb, dtype, "dbeta")
    if with_residual:
        helpers.assert_close(tdres, edx0, dtype, "dresidual")


def test_dropout_add_ln_checks(ops, cuda):
    import torch
    rows, cols = 8, 256
    x0 = torch.zeros(rows, cols, device=cuda)
    g = torch.ones(cols, device=cuda)
    z = torch.empty_like(x0)
    mu = torch.empty(rows, device=cuda)
    rs = torch.empty(rows, device=cuda)
    _sync_in()
    with pytest.raises(ops.AssertionError_, match="x must be given"):       # dropout keeps the pre-norm sum
        ops.dropout_add_ln_fwd(x0, None, g, None, z, None, mu, rs, 1e-6, True, dropout_p=0.1)
    with pytest.raises(ops.AssertionError_, match="dmask must be given"):
        ops.dropout_add_ln_fwd(x0, None, g, None, z, torch.empty_like(x0), mu, rs, 1e-6, True, dropout_p=0.1)
    with pytest.raises(ops.AssertionError_, match="z_subset"):
        ops.dropout_add_ln_fwd(x0, None, g, None, z, torch.empty_like(x0), mu, rs, 1e-6, True,
                               x0_subset=torch.ones(rows, dtype=torch.int32, device=cuda))
    with pytest.raises(ops.NotImplemented_, match="no kernel for weight dtype"):   # bf16 weights, fp32 input
        ops.dropout_add_ln_fwd(x0, None, g.bfloat16(), None, z, torch.empty_like(x0), mu, rs, 1e-6, True,
                               colscale=g.bfloat16())
    with pytest.raises(ops.AssertionError_, match="multiple of 8"):
        ops.dropout_add_ln_fwd(x0[:, :252].contiguous(), None, g[:252].contiguous(), None,
                               z[:, :252].contiguous(), None, mu, rs, 1e-6, True)
    with pytest.raises(ops.AssertionError_):     # x0 must be dense
        ops.dropout_add_ln_fwd(x0.t(), None, g, None, z, None, mu, rs, 1e-6, True)


MT19937_64_FIRST_OF_5489 = 14514284786278117030   # first output of std::mt19937_64 seeded with its default 5489


@pytest.mark.parametrize("is_rms", [False, True])
def test_dropout_add_ln_full_feature_set(ops, cuda, is_rms):
    """Dropout + rowscale + colscale + residual in fp32 with bf16 input through DropoutAddLnFwdCuda / BwdCuda.
    The seed comes from the layer's seeded generator, so the mask is known in advance."""
    import torch
    from oracle import dropout_add_ln as dal
    rows, cols, eps, p = 40, 1024, 1e-5, 0.2
    x0 = helpers.draw(1, (rows, cols), dtype="bf16"); residual = helpers.draw(2, (rows, cols), dtype="fp32")
    gamma = helpers.draw(3, (cols,), "uniform", 0.5, 1.5, "fp32"); beta = helpers.draw(4, (cols,), "normal", 0, 0.1, "fp32")
    rowscale = helpers.draw(5, (rows,), "uniform", 0.5, 2.0, "bf16")
    colscale = helpers.draw(6, (cols,), "uniform", 0.5, 2.0, "fp32")
    dz = helpers.draw(7, (rows, cols), dtype="bf16"); dx_in = helpers.draw(8, (rows, cols), dtype="fp32")
    emask = dal.dropout_keep(MT19937_64_FIRST_OF_5489, 0, rows * cols, np.float32(1) - np.float32(p)).reshape(rows, cols)
    ez, ex, emu, ers = dal.fwd(x0, residual, gamma, None if is_rms else beta, rowscale, colscale, dmask=emask,
                               dropout_p=p, eps=eps, is_rms=is_rms)
    tx0, trow, tdz = _dev((x0, rowscale, dz), "bf16", cuda)
    tres, tg, tb, tcol, tdxin = _dev((residual, gamma, beta, colscale, dx_in), "fp32", cuda)
    tz = torch.empty_like(tx0); tx = torch.empty_like(tres)
    tm = torch.zeros(rows, cols, dtype=torch.uint8, device=cuda)
    tmu = torch.empty(rows, device=cuda); trs = torch.empty(rows, device=cuda)
    _sync_in()
    ops.set_random_seed(5489)
    ops.dropout_add_ln_fwd(tx0, tres, tg, None if is_rms else tb, tz, tx, tmu, trs, eps, is_rms, dropout_p=p,
                           rowscale=trow, colscale=tcol, dmask=tm)
    ops.stream_sync()
    assert np.array_equal(tm.cpu().numpy(), emask)
    helpers.assert_close(tz, ez, "bf16", "z")
    helpers.assert_close(tx, ex, "fp32", "x")
    helpers.assert_close(trs, ers, "fp32", "rsigma")
    # the generator moves on: a second call draws another mask; reseeding brings the first one back
    tm2 = torch.zeros_like(tm)
    ops.dropout_add_ln_fwd(tx0, tres, tg, None if is_rms else tb, tz, tx, tmu, trs, eps, is_rms, dropout_p=p,
                           rowscale=trow, colscale=tcol, dmask=tm2)
    ops.stream_sync()
    assert 0.2 < (tm2 != tm).float().mean().item() < 0.45
    ops.set_random_seed(5489)
    ops.dropout_add_ln_fwd(tx0, tres, tg, None if is_rms else tb, tz, tx, tmu, trs, eps, is_rms, dropout_p=p,
                           rowscale=trow, colscale=tcol, dmask=tm2)
    ops.stream_sync()
    assert torch.equal(tm2, tm)

    xs = helpers.to_numpy(tx); mu32 = helpers.to_numpy(tmu); rs32 = helpers.to_numpy(trs)
    edx0, edres, edg, edb, edcol = dal.bwd(dz, dx_in, xs, x0, emask, mu32, rs32, gamma, rowscale, colscale,
                                           dropout_p=p, is_rms=is_rms)
    tdx0 = torch.empty_like(tx0); tdres = torch.empty_like(tres)
    tdg, tdb, tdcol = torch.empty_like(tg), torch.empty_like(tg), torch.empty_like(tg)
    _sync_in()
    ops.dropout_add_ln_bwd(tdz, tdxin, tx, tmu, trs, tg, tdx0, tdres, tdg, tdb, True, is_rms, dropout_p=p,
                           rowscale=trow, colscale=tcol, x0=tx0, dmask=tm, dcolscale=tdcol)
    ops.stream_sync()
    helpers.assert_close(tdx0, edx0, "bf16", "dx0")
    helpers.assert_close(tdres, edres, "fp32", "dresidual")
    helpers.assert_close(tdg, edg, "fp32", "dgamma")
    helpers.assert_close(tdb, edb, "fp32", "dbeta")
    helpers.assert_close(tdcol, edcol, "fp32", "dcolscale")


def test_dropout_add_ln_row_subsets(ops, cuda):
    import torch
    from oracle import dropout_add_ln as dal
    rows, x0_rows, z_rows, cols, eps, rsc = 12, 7, 5, 512, 1e-5, 0.5
    x0_subset = np.array([1, 0, 2, 3, 0, 4, 0, 5, 6, 0, 7, 0], dtype=np.int32)
    z_subset = np.array([0, 1, 0, 2, 3, 0, 4, 0, 0, 5, 0, 0], dtype=np.int32)
    x0 = helpers.draw(1, (x0_rows, cols), dtype="fp16"); residual = helpers.draw(2, (rows, cols), dtype="fp16")
    gamma = helpers.draw(3, (cols,), "uniform", 0.5, 1.5, "fp16"); beta = helpers.draw(4, (cols,), "normal", 0, 0.1, "fp16")
    dz = helpers.draw(5, (z_rows, cols), dtype="fp16")
    ez, ex, emu, ers = dal.fwd(x0, residual, gamma, beta, None, None, x0_subset, z_subset, None, 0.0, eps, rsc,
                               z_rows, False)
    tx0, tres, tg, tb, tdz = _dev((x0, residual, gamma, beta, dz), "fp16", cuda)
    sx0, sz = helpers.to_torch(x0_subset, "int32", cuda), helpers.to_torch(z_subset, "int32", cuda)
    tz = torch.empty(z_rows, cols, dtype=torch.float16, device=cuda); tx = torch.empty_like(tres)
    tmu = torch.empty(rows, device=cuda); trs = torch.empty(rows, device=cuda)
    _sync_in()
    ops.dropout_add_ln_fwd(tx0, tres, tg, tb, tz, tx, tmu, trs, eps, False, x0_subset=sx0, z_subset=sz,
                           rowscale_const=rsc, z_numrows=z_rows)
    ops.stream_sync()
    helpers.assert_close(tz, ez, "fp16", "z")
    helpers.assert_close(tx, ex, "fp16", "x")
    xs = helpers.to_numpy(tx); mu32 = helpers.to_numpy(tmu); rs32 = helpers.to_numpy(trs)
    edx0, edres, edg, edb, _ = dal.bwd(dz, None, xs, x0, None, mu32, rs32, gamma, None, None, x0_subset, z_subset,
                                       0.0, rsc, x0_rows, False)
    tdx0 = torch.empty_like(tx0); tdres = torch.empty_like(tres)
    tdg, tdb = torch.empty_like(tg), torch.empty_like(tg)
    _sync_in()
    ops.dropout_add_ln_bwd(tdz, None, tx, tmu, trs, tg, tdx0, tdres, tdg, tdb, True, False, x0_subset=sx0,
                           z_subset=sz, rowscale_const=rsc, x0_numrows=x0_rows)
    ops.stream_sync()
    helpers.assert_close(tdx0, edx0, "fp16", "dx0")
    helpers.assert_close(tdres, edres, "fp16", "dresidual")
    helpers.assert_close(tdg, edg, "fp16", "dgamma")
    helpers.assert_close(tdb, edb, "fp16", "dbeta")
    with pytest.raises(ops.AssertionError_, match="z must have shape"):
        ops.dropout_add_ln_fwd(tx0, tres, tg, tb, tz, tx, tmu, trs, eps, False, x0_subset=sx0, z_subset=sz,
                               rowscale_const=rsc, z_numrows=z_rows + 1)


@pytest.mark.parametrize("tied", [False, True])
def test_dropout_add_ln_parallel_residual(ops, cuda, tied):
    import torch
    from oracle import dropout_add_ln as dal
    rows, cols, eps, p = 24, 2048, 1e-5, 0.1
    dt = "bf16"
    x0 = helpers.draw(1, (rows, cols), dtype=dt); x1 = helpers.draw(2, (rows, cols), dtype=dt)
    residual = helpers.draw(3, (rows, cols), dtype=dt)
    g0 = helpers.draw(4, (cols,), "uniform", 0.5, 1.5, dt); b0 = helpers.draw(5, (cols,), "normal", 0, 0.1, dt)
    g1 = None if tied else helpers.draw(6, (cols,), "uniform", 0.5, 1.5, dt)
    b1 = None if tied else helpers.draw(7, (cols,), "normal", 0, 0.1, dt)
    dz0 = helpers.draw(8, (rows, cols), dtype=dt); dz1 = None if tied else helpers.draw(9, (rows, cols), dtype=dt)
    keep = np.float32(1) - np.float32(p)
    m0 = dal.dropout_keep(MT19937_64_FIRST_OF_5489, 0, rows * cols, keep, 0).reshape(rows, cols)
    m1 = dal.dropout_keep(MT19937_64_FIRST_OF_5489, 0, rows * cols, keep, 1).reshape(rows, cols)
    ez0, ez1, ex, emu, ers = dal.parallel_fwd(x0, x1, residual, g0, b0, g1, b1, m0, m1, p, eps, False)
    T = lambda a: None if a is None else helpers.to_torch(a, dt, cuda)
    tx0, tx1, tres, tg0, tb0, tg1, tb1, tdz0, tdz1 = map(T, (x0, x1, residual, g0, b0, g1, b1, dz0, dz1))
    tz0 = torch.empty_like(tx0); tz1 = None if tied else torch.empty_like(tx0); tx = torch.empty_like(tx0)
    tm0 = torch.zeros(rows, cols, dtype=torch.uint8, device=cuda); tm1 = torch.zeros_like(tm0)
    tmu = torch.empty(rows, device=cuda); trs = torch.empty(rows, device=cuda)
    _sync_in()
    ops.set_random_seed(5489)
    ops.dropout_add_ln_parallel_residual_fwd(tx0, tx1, tres, tg0, tb0, tg1, tb1, tz0, tz1, tx, tm0, tm1, tmu, trs,
                                             p, eps)
    ops.stream_sync()
    assert np.array_equal(tm0.cpu().numpy(), m0) and np.array_equal(tm1.cpu().numpy(), m1)
    helpers.assert_close(tz0, ez0, dt, "z0")
    if not tied:
        helpers.assert_close(tz1, ez1, dt, "z1")
    helpers.assert_close(tx, ex, dt, "x")
    xs = helpers.to_numpy(tx); mu32 = helpers.to_numpy(tmu); rs32 = helpers.to_numpy(trs)
    edx0, edx1, edres, edg0, edb0, edg1, edb1 = dal.parallel_bwd(dz0, dz1, None, xs, m0, m1, mu32, rs32, g0, g1, p,
                                                                 True, False)
    tdx0, tdx1, tdres = torch.empty_like(tx0), torch.empty_like(tx0), torch.empty_like(tx0)
    tdg0, tdb0 = torch.empty_like(tg0), torch.empty_like(tg0)
    tdg1 = None if tied else torch.empty_like(tg0); tdb1 = None if tied else torch.empty_like(tg0)
    _sync_in()
    ops.dropout_add_ln_parallel_residual_bwd(tdz0, tdz1, None, tx, tm0, tm1, tmu, trs, tg0, tg1, tdx0, tdx1, tdres,
                                             tdg0, tdb0, tdg1, tdb1, p, True, True)
    ops.stream_sync()
    helpers.assert_close(tdx0, edx0, dt, "dx0")
    helpers.assert_close(tdx1, edx1, dt, "dx1")
    helpers.assert_close(tdres, edres, dt, "dresidual")
    helpers.assert_close(tdg0, edg0, dt, "dgamma0")
    helpers.assert_close(tdb0, edb0, dt, "dbeta0")
    if not tied:
        helpers.assert_close(tdg1, edg1, dt, "dgamma1")
        helpers.assert_close(tdb1, edb1, dt, "dbeta1")


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape,dim", [((4, 6, 300), -1), ((5, 64, 33), 1), ((16, 2048), 1), ((7, 3, 5, 9), 0)])
def test_softmax_and_gradient(ops, cuda, dtype, shape, dim):
    import torch
    x = helpers.draw(51, shape, "normal", 0.0, 2.0, dtype)
    dy = helpers.draw(52, shape, dtype=dtype)
    ey = oracle.softmax_fwd(x, dim)
    tx, tdy = _dev((x, dy), dtype, cuda)
    ty = torch.empty_like(tx)
    _sync_in()
    ops.softmax(tx, ty, dim)
    ops.stream_sync()
    helpers.assert_close(ty, ey, dtype, "y")
    y_stored = helpers.to_numpy(ty)
    edx = oracle.softmax_bwd(y_stored, dy, dim)
    tdx = torch.empty_like(tx)
    _sync_in()
    ops.softmax_gradient(ty, tdy, tdx, dim)
    ops.stream_sync()
    helpers.assert_close(tdx, edx, dtype, "dx")


def test_softmax_of_a_permuted_view(ops, cuda):
    """Inputs and outputs of any stride are accepted: row-pitched ones go to the kernels as they are, any other
    input is made dense inside, any other output is written dense and laid over its strides afterwards."""
    import torch
    x = helpers.draw(61, (12, 40, 24), "normal", 0.0, 2.0, "fp32")
    tx = helpers.to_torch(x, "fp32", cuda).permute(2, 0, 1)       # [24, 12, 40], not dense
    ey = oracle.softmax_fwd(np.ascontiguousarray(x.transpose(2, 0, 1)), -1)
    ty = torch.empty((24, 12, 40), device=cuda)
    _sync_in()
    ops.softmax(tx, ty, -1)
    ops.stream_sync()
    helpers.assert_close(ty, ey, "fp32", "y")
    # the same into a permuted output
    base = torch.full((12, 40, 24), float("nan"), device=cuda)
    _sync_in()
    ops.softmax(tx, base.permute(2, 0, 1), -1)
    ops.stream_sync()
    helpers.assert_close(base.permute(2, 0, 1).contiguous(), ey, "fp32", "y")
    with pytest.raises(ops.AssertionError_, match="Invalid dimension"):
        ops.softmax(tx, ty, 3)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_outputs_of_any_layout(ops, cuda, dtype):
    """A transposed view, and a view with a stride between columns, as the output of LayerNorm forward / backward,
    softmax forward / backward (last and middle dimension), the cross-entropy gradients and a reduction: the
    values that land in the view equal the dense result bit for bit, and nothing outside the view is written."""
    import torch
    R, C = 37, 96
    x = helpers.draw(901, (R, C), dtype=dtype)
    dy = helpers.draw(902, (R, C), dtype=dtype)
    g = helpers.draw(903, (C,), "uniform", 0.5, 1.5, dtype)
    b = helpers.draw(904, (C,), "normal", 0.0, 0.1, dtype)
    tx, tdy, tg, tb = (helpers.to_torch(v, dtype, cuda) for v in (x, dy, g, b))
    td = tx.dtype

    def layouts():
        # (name, view of shape [R, C], its backing array, mask of the elements the view covers)
        t = torch.full((C, R), 7.0, dtype=td, device=cuda)
        yield "transposed", t.t(), t, torch.ones((C, R), dtype=torch.bool, device=cuda)
        w = torch.full((R, 2 * C), 7.0, dtype=td, device=cuda)
        m = torch.zeros((R, 2 * C), dtype=torch.bool, device=cuda)
        m[:, ::2] = True
        yield "every other column", w[:, ::2], w, m

    def check(run, what):
        dense = torch.empty((R, C), dtype=td, device=cuda)
        _sync_in()
        run(dense)
        ops.stream_sync()
        for name, view, backing, covered in layouts():
            assert not view.is_contiguous()
            _sync_in()
            run(view)
            ops.stream_sync()
            assert torch.equal(view.contiguous(), dense), "%s into a %s view" % (what, name)
            assert bool((backing[~covered] == 7.0).all()), "%s wrote outside a %s view" % (what, name)

    mean = torch.empty(R, dtype=torch.float32, device=cuda)
    rstd = torch.empty(R, dtype=torch.float32, device=cuda)
    check(lambda out: ops.fused_layer_norm(tx, tg, tb, mean, rstd, out, 1, 1e-5), "fused layer norm")
    dg, db = torch.empty_like(tg), torch.empty_like(tg)
    check(lambda out: ops.fused_layer_norm_gradient(tdy, tx, tg, tb, out, dg, db, mean, rstd, 1, 1e-5, False),
          "fused layer norm gradient")
    mean_t, var_t = torch.empty(R, dtype=td, device=cuda), torch.empty(R, dtype=td, device=cuda)
    check(lambda out: ops.layer_norm(tx, tg, tb, mean_t, var_t, out, 1, 1e-5), "layer norm")
    check(lambda out: ops.layer_norm_gradient(tdy, tx, tg, out, dg, db, mean_t, var_t, 1, 1e-5), "layer norm gradient")
    check(lambda out: ops.softmax(tx, out, -1), "softmax")
    check(lambda out: ops.softmax(tx, out, 0), "softmax over dimension 0")
    ty = torch.empty_like(tx)
    _sync_in()
    ops.softmax(tx, ty, -1)
    ops.stream_sync()
    check(lambda out: ops.softmax_gradient(ty, tdy, out, -1), "softmax gradient")
    labels = torch.randint(0, C, (R,), device=cuda, dtype=torch.int64)
    labels[3] = -100
    gl = helpers.to_torch(helpers.draw(905, (R,), dtype=dtype), dtype, cuda)
    check(lambda out: ops.softmax_cross_entropy_sparse_gradient(tx, labels, gl, out, -100), "sparse CE gradient")
    dense_labels = torch.softmax(tdy.float(), -1).to(td)
    check(lambda out: ops.softmax_cross_entropy_gradient(tx, dense_labels, gl, out), "dense CE gradient")
    x3 = helpers.to_torch(helpers.draw(906, (R, 5, C), dtype=dtype), dtype, cuda)
    check(lambda out: ops.reduce(x3, out, [1], "sum"), "sum over the middle dimension")


def test_row_pitched_views_reach_the_kernels_without_a_copy(ops, cuda):
    """Column slices of wider arrays (3-D here: [batch, seq, hidden] cut along hidden) as inputs AND outputs of the
    LayerNorm, Softmax and cross-entropy operators: results match the oracle, nothing outside the output slices is
    written, and the pool hands out no block for a dense copy (its allocation count only moves by the backward's
    scratch)."""
    import torch
    B, S, H, W, off = 3, 21, 512, 768, 128
    dt = "bf16"
    x = helpers.draw(81, (B, S, H), dtype=dt)
    dy = helpers.draw(82, (B, S, H), dtype=dt)
    g = helpers.draw(83, (H,), "uniform", 0.5, 1.5, dt)
    b = helpers.draw(84, (H,), "normal", 0.0, 0.1, dt)
    sent = 12288.0

    def wide(values=None):
        w = torch.full((B, S, W), sent, dtype=torch.bfloat16, device=cuda)
        if values is not None:
            w[:, :, off:off + H] = helpers.to_torch(values, dt, cuda)
        return w, w[:, :, off:off + H]

    def untouched(w):
        keep = torch.ones(W, dtype=torch.bool, device=cuda)
        keep[off:off + H] = False
        return bool((w[:, :, keep].float() == sent).all())

    _, sx = wide(x)
    _, sdy = wide(dy)
    wy, sy = wide()
    tg, tb = helpers.to_torch(g, dt, cuda), helpers.to_torch(b, dt, cuda)
    mean = torch.empty(B, S, 1, device=cuda)
    rstd = torch.empty(B, S, 1, device=cuda)
    _sync_in()
    before = ops.pool_stats()
    ops.fused_layer_norm(sx, tg, tb, mean, rstd, sy, 1, 1e-5)
    wp, sp = wide()
    ops.softmax(sx, sp, -1)
    ops.stream_sync()
    assert ops.pool_stats()["alloc_cnt"] == before["alloc_cnt"]          # no dense copy, no scratch
    x2, g64, b64 = x.reshape(-1, H), g, b
    ey, _, _, ers = oracle.layernorm_fwd(x2, g64, b64, 1e-5)
    helpers.assert_close(sy, ey.reshape(B, S, H), dt, "y")
    helpers.assert_close(rstd.reshape(-1), ers, "fp32", "rstd")
    helpers.assert_close(sp, oracle.softmax_fwd(x2).reshape(B, S, H), dt, "softmax")
    assert untouched(wy) and untouched(wp)
    wdx, sdx = wide()
    dg, db = torch.empty_like(tg), torch.empty_like(tb)
    mid = ops.pool_stats()
    ops.fused_layer_norm_gradient(sdy, sx, tg, tb, sdx, dg, db, mean, rstd, 1, 1e-5, False)
    wsm, ssm = wide()
    ops.softmax_gradient(sp, sdy, ssm, -1)
    ops.stream_sync()
    assert ops.pool_stats()["alloc_cnt"] - mid["alloc_cnt"] <= 1          # the backward's column-sum scratch only
    edx, edg, edb = oracle.layernorm_bwd(dy.reshape(-1, H), x2, g, helpers.to_numpy(mean).reshape(-1),
                                         helpers.to_numpy(rstd).reshape(-1), eps=1e-5, clamp_gamma=True)
    helpers.assert_close(sdx, edx.reshape(B, S, H), dt, "dx")
    helpers.assert_close(dg, edg, dt, "dgamma", scale=float(np.sqrt(B * S)))
    helpers.assert_close(ssm, oracle.softmax_bwd(helpers.to_numpy(sp).reshape(-1, H), dy.reshape(-1, H)).reshape(B, S, H),
                         dt, "softmax gradient")
    assert untouched(wdx) and untouched(wsm)
    # cross-entropy on logits padded along the class dimension, gradient written into a padded array
    lab = helpers.rng(85).integers(0, H, (B, S)).astype(np.int64)
    lab.reshape(-1)[::4] = -100
    tl = torch.from_numpy(lab).to(cuda)
    loss = torch.empty(B, S, dtype=torch.bfloat16, device=cuda)
    gl = helpers.draw(86, (B, S), "uniform", 0.5, 1.5, dt)
    wdl, sdl = wide()
    mid = ops.pool_stats()
    ops.softmax_cross_entropy_sparse(sx, tl, loss, -100)
    ops.softmax_cross_entropy_sparse_gradient(sx, tl, helpers.to_torch(gl, dt, cuda), sdl, -100)
    ops.stream_sync()
    assert ops.pool_stats()["alloc_cnt"] == mid["alloc_cnt"]
    helpers.assert_close(loss.reshape(-1), oracle.sce_sparse_fwd(x2, lab.reshape(-1), -100), dt, "loss")
    edl = oracle.sce_sparse_bwd(x2, lab.reshape(-1), gl.reshape(-1), -100)
    helpers.assert_close(sdl, edl.reshape(B, S, H), dt, "dlogits")
    assert untouched(wdl)
    # a view that is not row-pitched (every other column) still works as an input, through a dense copy
    half = torch.empty(B, S, H // 2, dtype=torch.bfloat16, device=cuda)
    ops.softmax(sx[:, :, ::2], half, -1)
    ops.stream_sync()
    helpers.assert_close(half, oracle.softmax_fwd(x2[:, ::2]).reshape(B, S, H // 2), dt, "softmax of strided columns")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_sparse_cross_entropy_and_gradient(ops, cuda, dtype):
    import torch
    shape, cols = (6, 11, 1000), 1000
    rows = 66
    ignored = -100
    x = helpers.draw(71, shape, "normal", 0.0, 3.0, dtype)
    g = helpers.rng(72)
    labels = g.integers(0, cols, size=shape[:-1]).astype(np.int64)
    labels.reshape(-1)[::7] = ignored
    gl = helpers.draw(73, shape[:-1], dtype=dtype)
    eloss = oracle.sce_sparse_fwd(x.reshape(rows, cols), labels.reshape(rows), ignored)
    egrad = oracle.sce_sparse_bwd(x.reshape(rows, cols), labels.reshape(rows), gl.reshape(rows), ignored)
    tx, tgl = _dev((x, gl), dtype, cuda)
    tl = torch.from_numpy(labels).to(cuda)
    tloss = torch.empty(shape[:-1], dtype=tx.dtype, device=cuda)
    tgrad = torch.empty_like(tx)
    _sync_in()
    ops.softmax_cross_entropy_sparse(tx, tl, tloss, ignored)
    ops.softmax_cross_entropy_sparse_gradient(tx, tl, tgl, tgrad, ignored)
    ops.stream_sync()
    helpers.assert_close(tloss.reshape(rows), eloss, dtype, "loss")
    helpers.assert_close(tgrad.reshape(rows, cols), egrad, dtype, "grad")
    got = helpers.to_numpy(tloss).reshape(rows)
    assert np.all(got[labels.reshape(rows) == ignored] == 0.0)
    assert np.all(helpers.to_numpy(tgrad).reshape(rows, cols)[labels.reshape(rows) == ignored] == 0.0)
    with pytest.raises(ops.AssertionError_, match="int64"):
        ops.softmax_cross_entropy_sparse(tx, tl.int(), tloss, ignored)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_dense_cross_entropy_and_gradient(ops, cuda, dtype):
    import torch
    rows, cols = 40, 777
    x = helpers.draw(81, (rows, cols), "normal", 0.0, 3.0, dtype)
    lab = helpers.rng(82).random((rows, cols)).astype(np.float32)
    lab = oracle.round_to(lab / lab.sum(axis=1, keepdims=True), dtype)
    gl = helpers.draw(83, (rows,), dtype=dtype)
    eloss = oracle.sce_dense_fwd(x, lab)
    egrad = oracle.sce_dense_bwd(x, lab, gl)
    tx, tlab, tgl = _dev((x, lab, gl), dtype, cuda)
    tloss = torch.empty(rows, dtype=tx.dtype, device=cuda)
    tgrad = torch.empty_like(tx)
    _sync_in()
    ops.softmax_cross_entropy(tx, tlab, tloss)
    ops.softmax_cross_entropy_gradient(tx, tlab, tgl, tgrad)
    ops.stream_sync()
    helpers.assert_close(tloss, eloss, dtype, "loss")
    helpers.assert_close(tgrad, egrad, dtype, "grad")


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp64", "int64"])
@pytest.mark.parametrize("axes", [[0], [1], [-1], [0, 2], [], [2, 0, 0]])
@pytest.mark.parametrize("red", ["sum", "mean"])
def test_reduce_kernel_entry(ops, cuda, dtype, axes, red):
    import torch
    shape = (9, 130, 24)
    if dtype == "int64":
        x = helpers.rng(91).integers(-1000, 1000, size=shape).astype(np.int64)
        tx = torch.from_numpy(x).to(cuda)
    else:
        x = helpers.draw(91, shape, dtype=dtype if dtype != "fp64" else "fp32")
        tx = helpers.to_torch(x, dtype, cuda)
    nd = len(shape)
    norm_axes = sorted(set(a % nd for a in axes)) if axes else list(range(nd))
    out_shape = [s for i, s in enumerate(shape) if i not in norm_axes] or [1]
    tout = torch.empty(out_shape, dtype=tx.dtype, device=cuda)
    _sync_in()
    ops.reduce(tx, tout, axes, red)
    ops.stream_sync()
    if dtype == "int64":
        e = x.sum(axis=tuple(norm_axes))
        if red == "mean":
            n = int(np.prod([shape[a] for a in norm_axes]))
            # integer mean: the sum times float(1/n), truncated back to the integer type
            e = (e.astype(np.float64) * float(np.float32(1.0) / np.float32(n))).astype(np.int64)
            assert np.all(np.abs(tout.cpu().numpy().reshape(e.shape) - e) <= 1)
        else:
            assert np.array_equal(tout.cpu().numpy().reshape(e.shape), e)
    else:
        e = oracle.reduce(x, norm_axes, red)
        # the mean is the sum times float(1/n): its factor carries fp32 rounding even for fp64 data
        rtol = 1e-6 if (dtype == "fp64" and red == "mean") else None
        helpers.assert_close(tout, np.asarray(e).reshape(out_shape), dtype, "%s over %s" % (red, axes), rtol=rtol)


def test_reduce_rejects_what_is_not_on_the_path(ops, cuda):
    import torch
    x = torch.ones(4, 8, device=cuda)
    _sync_in()
    out = torch.empty(8, device=cuda)
    x3, x2 = x * 3, x * 2
    _sync_in()
    ops.reduce(x3, out, [0], "max")
    ops.stream_sync()
    assert float(out.min()) == 3.0 and float(out.max()) == 3.0
    ops.reduce(x2, out, [0], "prod")
    ops.stream_sync()
    assert float(out.min()) == 16.0
    with pytest.raises(ops.NotImplemented_, match="none"):
        ops.reduce(x, torch.empty(8, device=cuda), [0], "none")
    with pytest.raises(ops.AssertionError_, match="Invalid dimension"):
        ops.reduce(x, torch.empty(8, device=cuda), [2], "sum")
    with pytest.raises(ops.AssertionError_, match="kept elements"):
        ops.reduce(x, torch.empty(5, device=cuda), [0], "sum")


def test_reduce_of_a_strided_view_needs_no_copy(ops, cuda):
    import torch
    x = helpers.draw(95, (64, 48, 20), dtype="fp32")
    tx = helpers.to_torch(x, "fp32", cuda)
    view = tx.permute(1, 2, 0)[:, ::2, :]            # [48, 10, 64], strides (20, 2, 960)
    e = np.ascontiguousarray(x.transpose(1, 2, 0)[:, ::2, :]).astype(np.float64).sum(axis=(0, 2))
    tout = torch.empty(10, device=cuda)
    before = ops.pool_stats()["alloc_cnt"]
    _sync_in()
    ops.reduce(view, tout, [0, 2], "sum")
    ops.stream_sync()
    helpers.assert_close(tout, e, "fp32", "strided sum")
    assert ops.pool_stats()["alloc_cnt"] - before <= 1      # at most the partials scratch, never a dense copy of x


def test_ndarray_statics_allocate_and_dispatch(ops, cuda):
    import torch
    dtype = "bf16"
    shape, cols = (8, 16, 1024), 1024
    rows = 128
    x, gamma, beta, _ = _norm_inputs(shape, cols, dtype, 400)
    tx, tg, tb = _dev((x, gamma, beta), dtype, cuda)
    _sync_in()
    # reduce: sum / mean with keepdims
    tsum = torch.empty((8, 1, 1024), dtype=tx.dtype, device=cuda)
    ops.ndarray_reduce(tx, "mean", [1], True, tsum)
    helpers.assert_close(tsum, np.asarray(oracle.reduce(x, [1], "mean")).reshape(8, 1, 1024), dtype, "mean")
    # softmax
    tsm = torch.empty_like(tx)
    ops.ndarray_softmax(tx, -1, tsm)
    helpers.assert_close(tsm, oracle.softmax_fwd(x, -1), dtype, "softmax")
    # layernorm (stats in the data dtype) and fused layernorm (fp32 stats)
    ey, emean, evar, erstd = oracle.layernorm_fwd(x.reshape(rows, cols), gamma, beta, 1e-5)
    ty = torch.empty_like(tx)
    tmean = torch.empty((8, 16, 1), dtype=tx.dtype, device=cuda)
    tvar = torch.empty((8, 16, 1), dtype=tx.dtype, device=cuda)
    ops.ndarray_layernorm(tx, tg, tb, 1, 1e-5, False, ty, tmean, tvar)
    helpers.assert_close(ty, ey.reshape(shape), dtype, "layernorm")
    helpers.assert_close(tvar.reshape(rows), evar, dtype, "var")
    tmean32 = torch.empty((8, 16, 1), dtype=torch.float32, device=cuda)
    trstd32 = torch.empty((8, 16, 1), dtype=torch.float32, device=cuda)
    ops.ndarray_layernorm(tx, tg, tb, 1, 1e-5, True, ty, tmean32, trstd32)
    helpers.assert_close(ty, ey.reshape(shape), dtype, "fused layernorm")
    helpers.assert_close(trstd32.reshape(rows), erstd, "fp32", "rstd")


@pytest.mark.parametrize("reduction", ["mean", "sum", "none"])
def test_ndarray_sceloss_reductions(ops, cuda, reduction):
    """kMEAN divides by ALL rows, ignored ones included (it is a plain mean over the per-row losses)."""
    import torch
    rows, cols, ignored = 96, 512, -1
    x = helpers.draw(500, (rows, cols), "normal", 0.0, 2.0, "fp32")
    labels = helpers.rng(501).integers(0, cols, size=rows).astype(np.int64)
    labels[::5] = ignored
    per_row = oracle.sce_sparse_fwd(x, labels, ignored)
    tx = helpers.to_torch(x, "fp32", cuda)
    tl = torch.from_numpy(labels).to(cuda)
    _sync_in()
    if reduction == "none":
        out = torch.empty(rows, device=cuda)
        ops.ndarray_sceloss(tx, tl, out, "none", ignored_index=ignored)
        helpers.assert_close(out, per_row, "fp32", "per-row loss")
    else:
        out = torch.empty(1, device=cuda)
        ops.ndarray_sceloss(tx, tl, out, reduction, ignored_index=ignored)
        e = per_row.sum() / rows if reduction == "mean" else per_row.sum()
        helpers.assert_close(out, np.array([e]), "fp32", reduction)
    # dense labels through the same static
    lab = np.zeros((rows, cols), dtype=np.float32)
    keep = labels != ignored
    lab[np.arange(rows)[keep], labels[keep]] = 1.0
    out = torch.empty(rows, device=cuda)
    ops.ndarray_sceloss(tx, helpers.to_torch(lab, "fp32", cuda), out, "none")
    helpers.assert_close(out, per_row, "fp32", "one-hot dense labels equal sparse labels")


def test_empty_arrays_are_no_ops(ops, cuda):
    import torch
    x = torch.empty((0, 64), device=cuda)
    g = torch.ones(64, device=cuda)
    _sync_in()
    ops.softmax(x, torch.empty_like(x), -1)
    ops.layer_norm(x, g, g, torch.empty((0, 1), device=cuda), torch.empty((0, 1), device=cuda),
                   torch.empty_like(x), 1, 1e-5)
    dg = torch.full((64,), 7.0, device=cuda)
    db = torch.full((64,), 7.0, device=cuda)
    _sync_in()
    ops.layer_norm_gradient(x, x, g, torch.empty_like(x), dg, db, torch.empty((0, 1), device=cuda),
                            torch.empty((0, 1), device=cuda), 1, 1e-5)
    ops.stream_sync()
    assert float(dg.abs().sum()) == 0.0 and float(db.abs().sum()) == 0.0     # empty column sums
    ops.softmax_cross_entropy_sparse(x, torch.empty(0, dtype=torch.int64, device=cuda),
                                     torch.empty(0, device=cuda), -1)
    out = torch.full((64,), 3.0, device=cuda)
    _sync_in()
    ops.reduce(x, out, [0], "sum")
    ops.stream_sync()
    assert float(out.abs().sum()) == 0.0


def test_device_pool_reuses_and_orders_across_streams(ops, cuda):
    """The real pool on the GPU: same-stream reuse, cross-stream take, parking, EmptyCache."""
    ops.synchronize_all()
    ops.pool_empty_cache()
    s0 = ops.pool_stats()
    a = ops.pool_alloc(5 << 20, stream=1)
    assert a.ptr % 256 == 0 and a.size == 5 << 20
    ops.pool_free(a)
    b = ops.pool_alloc(5 << 20, stream=1)
    assert b.ptr == a.ptr
    ops.pool_free(b)
    c = ops.pool_alloc(5 << 20, stream=2)                # taken from stream 1's cache behind an event
    assert c.ptr == a.ptr
    ops.pool_mark_used(c, 3)
    ops.pool_free(c)                                     # parked behind an event on stream 3 (idle: passes at once)
    d = ops.pool_alloc(5 << 20, stream=2)
    s1 = ops.pool_stats()
    assert s1["segment_allocs"] - s0["segment_allocs"] <= 2
    assert s1["cross_stream_takes"] - s0["cross_stream_takes"] >= 1
    assert s1["parked"] - s0["parked"] == 1
    ops.pool_free(d)
    small = [ops.pool_alloc(1000, stream=1) for _ in range(8)]
    assert len({blk.ptr for blk in small}) == 8
    assert max(blk.ptr for blk in small) - min(blk.ptr for blk in small) < (2 << 20)    # one segment
    for blk in small:
        ops.pool_free(blk)
    with pytest.raises(ops.ValueError_, match="freed twice"):
        ops.pool_free(small[0])
    ops.pool_empty_cache()
    s2 = ops.pool_stats()
    assert s2["allocated"] == 0 and s2["reserved"] == 0


def test_operators_leave_no_memory_behind(ops, cuda):
    import torch
    x = torch.randn(256, 4096, device=cuda, dtype=torch.bfloat16)
    g = torch.ones(4096, device=cuda, dtype=torch.bfloat16)
    dx, dg, db = torch.empty_like(x), torch.empty_like(g), torch.empty_like(g)
    mu = torch.empty(256, device=cuda)
    rs = torch.empty(256, device=cuda)
    z = torch.empty_like(x)
    _sync_in()
    for _ in range(3):
        ops.dropout_add_ln_fwd(x, None, g, None, z, None, mu, rs, 1e-6, True)
        ops.dropout_add_ln_bwd(x, None, x, mu, rs, g, dx, None, dg, db, False, True)
    ops.stream_sync()
    s = ops.pool_stats()
    assert s["allocated"] == 0                 # scratch went back to the pool
    assert s["cache_hits"] >= 2                # and was reused by the later iterations


def test_two_streams_share_the_pool_without_corruption(ops, cuda):
    """Operators alternate between two of the layer's streams while their scratch and temporaries come
    from the same pool: blocks freed on one stream are taken by the other behind an event.  Every result
    is checked, so a block reused before its previous user finished would show up as a wrong answer."""
    import torch
    rows, cols = 2048, 4096
    xs = [helpers.draw(700 + i, (rows, cols), dtype="bf16") for i in range(2)]
    dys = [helpers.draw(710 + i, (rows, cols), dtype="bf16") for i in range(2)]
    gamma = helpers.draw(720, (cols,), "uniform", 0.8, 1.2, "bf16")
    want = []
    for x, dy in zip(xs, dys):
        z, _, mu, rs = oracle.dropout_add_ln_fwd(x, None, gamma, None, 1e-6, True)
        dx0, dg, _ = oracle.dropout_add_ln_bwd(dy, None, x, mu.astype(np.float32), rs.astype(np.float32), gamma, True)
        want.append((z, dx0, dg, np.asarray(oracle.reduce(x, [0], "sum"))))
    tg = helpers.to_torch(gamma, "bf16", cuda)
    dev = []
    for x, dy in zip(xs, dys):
        tx, tdy = helpers.to_torch(x, "bf16", cuda), helpers.to_torch(dy, "bf16", cuda)
        dev.append(dict(x=tx, dy=tdy, z=torch.empty_like(tx), dx=torch.empty_like(tx), dg=torch.empty_like(tg),
                        db=torch.empty_like(tg), mu=torch.empty(rows, device=cuda), rs=torch.empty(rows, device=cuda),
                        colsum=torch.empty(cols, dtype=tx.dtype, device=cuda)))
    _sync_in()
    before = ops.pool_stats()
    for it in range(6):
        for k, stream in enumerate((1, 2)):
            d = dev[(k + it) % 2]          # the two data sets swap streams every iteration
            ops.dropout_add_ln_fwd(d["x"], None, tg, None, d["z"], None, d["mu"], d["rs"], 1e-6, True, stream=stream)
            ops.dropout_add_ln_bwd(d["dy"], None, d["x"], d["mu"], d["rs"], tg, d["dx"], None, d["dg"], d["db"],
                                   False, True, stream=stream)
            ops.reduce(d["x"], d["colsum"], [0], "sum", stream=stream)
        ops.stream_sync(1)
        ops.stream_sync(2)
    for d, (z, dx0, dg, colsum) in zip(dev, want):
        helpers.assert_close(d["z"], z, "bf16", "z")
        helpers.assert_close(d["dx"], dx0, "bf16", "dx0")
        helpers.assert_close(d["dg"], dg, "bf16", "dgamma")
        helpers.assert_close(d["colsum"], colsum, "bf16", "column sums", scale=float(np.sqrt(rows)))
    after = ops.pool_stats()
    assert after["allocated"] == before["allocated"]
    assert after["segment_allocs"] - before["segment_allocs"] <= 6      # scratch is recycled, not re-allocated


def test_native_cpp_gpu_selftest(cuda):
    """tests/cpp/gpu_selftest.cc: the layer driven from C++ (NDArray::cuda / cpu / zeros, the operator
    statics, events, the pool) and checked against double-precision loops inside the binary."""
    import os
    import subprocess
    exe = os.path.join(helpers.ROOT, "hotspa-ae_amd", "lib", "hetu_gpu_selftest")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    failed = [l for l in proc.stdout.splitlines() if l.startswith("[FAIL]")]
    assert proc.returncode == 0 and not failed, proc.stdout[-4000:]
    assert sum(l.startswith("[ OK ]") for l in proc.stdout.splitlines()) >= 8


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(3, 5, 16, 16), (2, 4, 28, 36), (1, 2, 7, 9)])
def test_instance_norm_and_gradient(ops, cuda, dtype, shape):
    """An instance norm is a layer norm without scale and bias over each [H, W] plane."""
    import torch
    n, c, h, w = shape
    rows, cols, eps = n * c, h * w, 1e-5
    x = helpers.draw(800 + cols, shape, "normal", 0.5, 2.0, dtype)
    dy = helpers.draw(801 + cols, shape, dtype=dtype)
    ones, zeros = np.ones(cols, np.float32), np.zeros(cols, np.float32)
    ey, emean, evar, erstd = oracle.layernorm_fwd(x.reshape(rows, cols), ones, zeros, eps)
    tx, tdy = _dev((x, dy), dtype, cuda)
    ty = torch.empty_like(tx)
    tmean = torch.empty((n, c, 1, 1), dtype=tx.dtype, device=cuda)
    tvar = torch.empty((n, c, 1, 1), dtype=tx.dtype, device=cuda)
    _sync_in()
    ops.instance_norm(tx, tmean, tvar, ty, eps)
    ops.stream_sync()
    helpers.assert_close(ty, ey.reshape(shape), dtype, "y")
    helpers.assert_close(tvar.reshape(rows), evar, dtype, "var")
    mean_r = helpers.to_numpy(tmean).reshape(rows).astype(np.float64)
    rstd_r = 1.0 / np.sqrt(helpers.to_numpy(tvar).reshape(rows).astype(np.float64) + eps)
    edx, _, _ = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), ones, mean_r.astype(np.float32),
                                     rstd_r.astype(np.float32))
    tdx = torch.empty_like(tx)
    before = ops.pool_stats()["alloc_cnt"]
    _sync_in()
    ops.instance_norm_gradient(tdy, tx, tdx, tmean, tvar, eps)
    ops.stream_sync()
    helpers.assert_close(tdx, edx.reshape(shape), dtype, "dx")
    assert ops.pool_stats()["alloc_cnt"] == before          # no column sums, so no scratch
    with pytest.raises(ops.AssertionError_, match="N, C, H, W"):
        ops.instance_norm(tx.reshape(n * c, h, w), tmean, tvar, ty.reshape(n * c, h, w), eps)


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
def test_elementwise_entry_points(ops, cuda, dtype):
    """AddElewiseCuda ... DivElewiseCuda with a per-row operand, the ...ConstCuda entries (constant on the left),
    ExpCuda / LogCuda / OppositeCuda / SqrtCuda."""
    import torch
    rows, cols = 50, 768
    a = oracle.round_to(np.abs(helpers.draw(1, (rows, cols))) + np.float32(0.5), dtype)
    b = oracle.round_to(np.abs(helpers.draw(2, (rows, 1))) + np.float32(0.5), dtype)
    ta, tb = _dev((a, b), dtype, cuda)
    out = torch.empty_like(ta)
    npf = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    ad, bd = a.astype(np.float64), b.astype(np.float64)
    _sync_in()
    for op, f in npf.items():
        ops.binary(op, ta, tb, out)
        ops.stream_sync()
        helpers.assert_close(out, f(ad, bd), dtype, op)
        ops.binary(op, tb, ta, out)                       # the broadcast operand on the left
        ops.stream_sync()
        helpers.assert_close(out, f(bd, ad), dtype, op + " swapped")
    c = 1.5
    for op, f in npf.items():                             # the constant is the left operand
        ops.binary_const(op, ta, c, out)
        ops.stream_sync()
        helpers.assert_close(out, f(c, ad), dtype, op + " const")
    for op, f in {"exp": np.exp, "log": np.log, "neg": np.negative, "sqrt": np.sqrt}.items():
        ops.unary(op, ta, out)
        ops.stream_sync()
        helpers.assert_close(out, f(ad), dtype, op)
    with pytest.raises(ops.AssertionError_, match="Divided by 0"):
        ops.binary_const("div", ta, 0.0, out)
    with pytest.raises(ops.AssertionError_, match="broadcast"):
        ops.binary("add", ta, ta[:, :cols - 1], out)
    with pytest.raises(ops.NotImplemented_):
        ops.unary("exp", ta.long(), out.long())


def test_ndarray_elementwise_statics(ops, cuda):
    """NDArray::add / sub / mul / div / exp / log / neg / sqrt: results from the pool, and in place."""
    import torch
    a = torch.rand(33, 1000, device=cuda) + 0.5
    b = torch.rand(33, 1, device=cuda) + 0.5
    out = torch.empty_like(a)
    _sync_in()
    for op, f in {"add": torch.add, "sub": torch.sub, "mul": torch.mul, "div": torch.div}.items():
        ops.ndarray_binary(op, a, b, out)
        assert torch.allclose(out, f(a, b), rtol=1e-6, atol=0)
    for op, f in {"exp": torch.exp, "log": torch.log, "neg": torch.neg, "sqrt": torch.sqrt}.items():
        ops.ndarray_unary(op, a, out)
        assert torch.allclose(out, f(a), rtol=1e-6, atol=1e-7)
    want = a / b
    ops.ndarray_binary("div", a, b, in_place=True)
    ops.stream_sync()
    assert torch.allclose(a, want, rtol=1e-6, atol=0)
    want = torch.log(a)
    ops.ndarray_unary("log", a, in_place=True)
    ops.stream_sync()
    assert torch.allclose(a, want, rtol=1e-6, atol=1e-7)
    t3 = torch.rand(4, 5, 6, device=cuda)
    out3 = torch.empty(4, 5, 6, device=cuda)
    ops.ndarray_binary("mul", t3, torch.rand(5, 1, device=cuda).add_(1.0), out3)
    with pytest.raises(ops.AssertionError_, match="cannot be broadcast"):
        ops.ndarray_binary("add", t3, torch.rand(4, 5, device=cuda), out3)


def test_vocab_parallel_cross_entropy_entry_points(ops, cuda):
    import torch
    rows, cols, start, ignored = 64, 2048, 4096, -100
    g = helpers.rng(3)
    logits = helpers.draw(4, (rows, cols), dtype="bf16")
    labels = g.integers(start - cols, start + 2 * cols, rows).astype(np.int64); labels[5] = ignored
    tl = helpers.to_torch(logits, "bf16", cuda); tlab = torch.from_numpy(labels).to(cuda)
    picked = torch.full((rows, 1), 9.0, dtype=torch.bfloat16, device=cuda)
    lse = torch.full((rows, 1), 3.0, dtype=torch.bfloat16, device=cuda)
    _sync_in()
    ops.vocab_parallel_cross_entropy(tl, tlab, start, start + cols, ignored, picked, lse)
    ops.stream_sync()
    inside = (labels >= start) & (labels < start + cols)
    want = np.where(inside, logits[np.arange(rows), np.clip(labels - start, 0, cols - 1)], 0.0)
    assert np.array_equal(helpers.to_numpy(picked).reshape(rows), want)
    assert np.array_equal(helpers.to_numpy(lse).reshape(rows), np.where(labels == ignored, 0.0, 3.0))
    sm = torch.softmax(tl.float(), dim=1).bfloat16()
    gl = torch.rand(rows, 1, device=cuda).bfloat16()
    out = torch.empty_like(sm)
    _sync_in()
    ops.vocab_parallel_cross_entropy_gradient(sm, tlab, start, start + cols, ignored, gl, out)
    ops.stream_sync()
    onehot = np.zeros((rows, cols)); onehot[np.flatnonzero(inside), (labels - start)[inside]] = 1.0
    helpers.assert_close(out, (helpers.to_numpy(sm).astype(np.float64) - onehot) * helpers.to_numpy(gl), "bf16", "grad")
    with pytest.raises(ops.AssertionError_, match="does not match"):
        ops.vocab_parallel_cross_entropy(tl, tlab, start, start + cols - 1, ignored, picked, lse)
    with pytest.raises(ops.AssertionError_, match="int64"):
        ops.vocab_parallel_cross_entropy(tl, tlab.int(), start, start + cols, ignored, picked, lse)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("p", [1, 2, 3])
def test_norm_and_gradient_entry_points(ops, cuda, dtype, p):
    import torch
    shape, dim = (6, 40, 64), -2
    x = helpers.draw(70 + p, shape, dtype=dtype)
    want = oracle.norm_p_fwd(x, 1, p)
    tx = helpers.to_torch(x, dtype, cuda)
    out = torch.empty(6, 64, dtype=tx.dtype, device=cuda)
    _sync_in()
    ops.norm(tx, out, dim, p)
    ops.stream_sync()
    helpers.assert_close(out, want, dtype, "norm")
    keep = torch.empty(6, 1, 64, dtype=tx.dtype, device=cuda)
    ops.ndarray_norm(tx, p, dim, True, keep)              # NDArray::norm with keepdim
    assert torch.equal(keep.view(6, 64), out)
    grad = helpers.draw(80, (6, 64), dtype=dtype)
    want_g = oracle.norm_p_bwd(x, helpers.to_numpy(out).astype(np.float64), grad, 1, p)
    dx = torch.empty_like(tx)
    _sync_in()
    ops.norm_gradient(tx, out, helpers.to_torch(grad, dtype, cuda), dx, dim, p)
    ops.stream_sync()
    helpers.assert_close(dx, want_g, dtype, "gradient")
    # a permuted view as input: the forward plans on strides, the gradient makes its operands dense
    tv = tx.permute(2, 0, 1)
    out2 = torch.empty(64, 6, dtype=tx.dtype, device=cuda)
    ops.norm(tv, out2, 2, p)
    ops.stream_sync()
    helpers.assert_close(out2, want.T, dtype, "norm of a view")
    with pytest.raises(ops.ValueError_, match="at least 1"):
        ops.norm(tx, out, dim, 0)
    with pytest.raises(ops.AssertionError_, match="does not hold"):
        ops.norm(tx, out[:, :63].contiguous(), dim, p)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_batch_norm_entry_points(ops, cuda, dtype):
    import torch
    shape = (6, 12, 10, 10)
    g = helpers.rng(91)
    x = oracle.round_to((g.standard_normal(shape) * 2 + 1).astype(np.float32), dtype)
    scale = g.uniform(0.5, 1.5, 12).astype(np.float32); bias = g.standard_normal(12).astype(np.float32)
    rm = g.standard_normal(12).astype(np.float32); rv = g.uniform(0.5, 2, 12).astype(np.float32)
    dy = oracle.round_to(g.standard_normal(shape).astype(np.float32), dtype)
    ey, erm, erv, emean, einv = oracle.batch_norm_fwd(x, scale, bias, rm, rv, 0.1, 1e-5)
    tx = helpers.to_torch(x, dtype, cuda)
    ts, tb, trm, trv = _dev((scale, bias, rm, rv), "fp32", cuda)
    ty = torch.empty_like(tx); sm = torch.empty_like(ts); sv = torch.empty_like(ts)
    _sync_in()
    ops.batch_norm(tx, ts, tb, ty, 0.1, 1e-5, trm, trv, sm, sv)
    ops.stream_sync()
    helpers.assert_close(ty, ey, dtype, "y")
    helpers.assert_close(trm, erm, "fp32", "running_mean", scale=1.0)
    helpers.assert_close(trv, erv, "fp32", "running_var", rtol=1e-4)
    helpers.assert_close(sv, einv, "fp32", "save_var (inverse standard deviation)", rtol=1e-4)
    edx, eds, edb = oracle.batch_norm_bwd(dy, x, scale, helpers.to_numpy(sm), helpers.to_numpy(sv))
    dx = torch.empty_like(tx); ds = torch.empty_like(ts); db = torch.empty_like(ts)
    _sync_in()
    ops.batch_norm_gradient(helpers.to_torch(dy, dtype, cuda), tx, ts, dx, ds, db, 1e-5, sm, sv)
    ops.stream_sync()
    helpers.assert_close(dx, edx, dtype, "dx", rtol=2e-2 if dtype == "bf16" else 1e-4)
    helpers.assert_close(ds, eds, "fp32", "dscale", rtol=1e-4)
    helpers.assert_close(db, edb, "fp32", "dbias", rtol=1e-4)
    if dtype == "bf16":
        with pytest.raises(ops.AssertionError_, match="bn_scale must have dtype"):
            ops.batch_norm(tx, ts.bfloat16(), tb, ty, 0.1, 1e-5, trm, trv, sm, sv)
    with pytest.raises(ops.AssertionError_, match="one value per channel"):
        ops.batch_norm(tx, ts[:11].contiguous(), tb, ty, 0.1, 1e-5, trm, trv, sm, sv)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_permuted_views_run_in_place(ops, cuda, dtype):
    """x.permute(0, 2, 1, 3) of a dense [B, H, S, D] array as input AND output of the norm / softmax / cross-entropy
    operators: the values equal the dense call's bit for bit, and the operator takes nothing from the pool for the
    forward calls (no gather of the input, no stand-in for the output: the reference reads such views through its
    OffsetCalculator, this layer through the row levels of the kernels)."""
    import torch
    B, H, S, D = 2, 3, 5, 256
    x = helpers.draw(951, (B, S, H, D), dtype=dtype)           # the VIEW's logical contents
    dy = helpers.draw(952, (B, S, H, D), dtype=dtype)
    g = helpers.draw(953, (D,), "uniform", 0.5, 1.5, dtype)
    b = helpers.draw(954, (D,), "normal", 0.0, 0.1, dtype)
    tg, tb = helpers.to_torch(g, dtype, cuda), helpers.to_torch(b, dtype, cuda)
    td = tg.dtype
    rows = B * S * H

    def permuted(values):
        stored = helpers.to_torch(np.ascontiguousarray(np.transpose(values, (0, 2, 1, 3))), dtype, cuda)   # [B, H, S, D]
        return stored.permute(0, 2, 1, 3)

    def empty_view():
        return torch.full((B, H, S, D), 7.0, dtype=td, device=cuda).permute(0, 2, 1, 3)

    vx, vdy = permuted(x), permuted(dy)
    dx_dense, dy_dense = vx.contiguous(), vdy.contiguous()
    assert not vx.is_contiguous()

    def both(run, what, allocs=0, exact=True):
        """run(x_like, dy_like, out) on dense arrays, then on the views; allocs = pool allocations the call may make;
        exact=False where the view takes another instance of the kernel than the dense array (the walking backward
        kernel splits row numbers in its general instance only), whose results may differ in the last bit"""
        dense = torch.empty((B, S, H, D), dtype=td, device=cuda)
        _sync_in()
        run(dx_dense, dy_dense, dense)
        ops.stream_sync()
        view = empty_view()
        _sync_in()
        before = ops.pool_stats()["alloc_cnt"]
        run(vx, vdy, view)
        ops.stream_sync()
        assert ops.pool_stats()["alloc_cnt"] - before == allocs, what + ": pool allocations for a permuted view"
        if exact:
            assert torch.equal(view.contiguous(), dense), what
        else:
            helpers.assert_close(view.contiguous(), helpers.to_numpy(dense).astype(np.float64), dtype, what)

    mean = torch.empty(rows, dtype=torch.float32, device=cuda)
    rstd = torch.empty(rows, dtype=torch.float32, device=cuda)
    both(lambda a, d, out: ops.fused_layer_norm(a, tg, tb, mean, rstd, out, 1, 1e-5), "fused layer norm")
    ey, em, _, ers = oracle.layernorm_fwd(x.reshape(rows, D), g, b, 1e-5)
    helpers.assert_close(rstd, ers, "fp32", "rstd")
    dg, db = torch.empty_like(tg), torch.empty_like(tg)
    # the backward takes its column-sum partials from the pool: one allocation, views or not
    both(lambda a, d, out: ops.fused_layer_norm_gradient(d, a, tg, tb, out, dg, db, mean, rstd, 1, 1e-5, False),
         "fused layer norm gradient", allocs=1, exact=False)
    edx, _, _ = oracle.layernorm_bwd(dy.reshape(rows, D), x.reshape(rows, D), g, helpers.to_numpy(mean),
                                     helpers.to_numpy(rstd), eps=1e-5, clamp_gamma=True)
    view = empty_view()
    _sync_in()
    ops.fused_layer_norm_gradient(vdy, vx, tg, tb, view, dg, db, mean, rstd, 1, 1e-5, False)
    ops.stream_sync()
    helpers.assert_close(view.reshape(rows, D), edx, dtype, "dx")
    mean_t, var_t = torch.empty(rows, dtype=td, device=cuda), torch.empty(rows, dtype=td, device=cuda)
    both(lambda a, d, out: ops.layer_norm(a, tg, tb, mean_t, var_t, out, 1, 1e-5), "layer norm")
    both(lambda a, d, out: ops.layer_norm_gradient(d, a, tg, out, dg, db, mean_t, var_t, 1, 1e-5), "layer norm gradient",
         allocs=1, exact=False)
    both(lambda a, d, out: ops.softmax(a, out, -1), "softmax")
    ty = torch.empty((B, S, H, D), dtype=td, device=cuda)
    _sync_in()
    ops.softmax(dx_dense, ty, -1)
    ops.stream_sync()
    vy = permuted(helpers.to_numpy(ty))
    dense = torch.empty((B, S, H, D), dtype=td, device=cuda)
    view = empty_view()
    _sync_in()
    ops.softmax_gradient(ty, dy_dense, dense, -1)
    before = ops.pool_stats()["alloc_cnt"]
    ops.softmax_gradient(vy, vdy, view, -1)
    ops.stream_sync()
    assert ops.pool_stats()["alloc_cnt"] == before and torch.equal(view.contiguous(), dense), "softmax gradient"
    labels = torch.randint(0, D, (B, S, H), device=cuda, dtype=torch.int64)
    labels[0, 1, 2] = -100
    gl = helpers.to_torch(helpers.draw(955, (B, S, H), dtype=dtype), dtype, cuda)
    loss_d = torch.empty((B, S, H), dtype=td, device=cuda)
    loss_v = torch.empty((B, S, H), dtype=td, device=cuda)
    _sync_in()
    ops.softmax_cross_entropy_sparse(dx_dense, labels, loss_d, -100)
    before = ops.pool_stats()["alloc_cnt"]
    ops.softmax_cross_entropy_sparse(vx, labels, loss_v, -100)
    ops.stream_sync()
    assert ops.pool_stats()["alloc_cnt"] == before and torch.equal(loss_v, loss_d), "sparse CE"
    both(lambda a, d, out: ops.softmax_cross_entropy_sparse_gradient(a, labels, gl, out, -100), "sparse CE gradient")
