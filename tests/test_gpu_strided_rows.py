"""Views with permuted leading dimensions (x.permute(0, 2, 1, 3) of a [B, H, S, D] array and the like: rows stay
contiguous, the leading dimensions do not step by one pitch) go through the *_strided_rows entry points as they
are: read and written in place on a three-dimensional grid, no gather before and no scatter after.  Every result is
compared with the oracle on the view's logical contents and, bit for bit, with the same call on dense copies;
inputs are left untouched and an output view that is itself a slice of a padded buffer leaves the padding alone."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

SENTINEL = 12288.0          # exactly representable in bf16

# (stored shape, permutation of the leading dimensions, columns): the view is stored.permute(perm + (last,))
#   [B, H, S, D] -> [B, S, H, D]: three levels;  [S, H, D] -> [H, S, D]: two levels;
#   [A, B, C, D] -> [C, B, A, D]: three levels, all reversed;  row counts that are odd and one that is 1
VIEWS = [((2, 4, 6, 1024), (0, 2, 1)), ((5, 3, 4096), (1, 0)), ((3, 2, 5, 512), (2, 1, 0)), ((1, 7, 3, 2048), (0, 2, 1)),
         ((2, 3, 1, 5120), (1, 0, 2)), ((4, 33, 256), (1, 0)), ((2, 2, 3, 264), (0, 2, 1)),
         # more rows than the walking backward kernel has workgroups times ring slots: its steady loop and its tail
         ((40, 33, 4096), (1, 0)), ((3, 7, 61, 2048), (0, 2, 1))]


def _view(values, perm, dt, dev, pad=0):
    """The stored array (optionally with `pad` extra sentinel columns per row) on the device and its permuted view;
    `values` is given in the VIEW's logical order."""
    import torch
    nd = values.ndim
    inv = np.argsort(perm).tolist() + [nd - 1]
    stored = np.ascontiguousarray(np.transpose(values, inv))
    t = helpers.to_torch(stored, dt, dev)
    if pad:
        wide = torch.full(tuple(stored.shape[:-1]) + (stored.shape[-1] + pad,), SENTINEL, dtype=t.dtype, device=dev)
        wide[..., :stored.shape[-1]] = t
        t = wide[..., :stored.shape[-1]]
    else:
        wide = t
    return wide, t.permute(*perm, nd - 1)


def _out_view(shape_view, perm, dt, dev, pad=0):
    import torch
    nd = len(shape_view)
    inv = np.argsort(perm).tolist()
    stored_shape = [shape_view[i] for i in inv] + [shape_view[-1] + pad]
    wide = torch.full(stored_shape, SENTINEL, dtype=helpers.load_package().torch_dtype(dt), device=dev)
    t = wide[..., :shape_view[-1]]
    return wide, t.permute(*perm, nd - 1)


def _padding_untouched(wide, cols):
    return bool((wide[..., cols:].float() == SENTINEL).all())


def _shape_of_view(stored, perm):
    return tuple(stored[i] for i in perm) + (stored[-1],)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("case", VIEWS, ids=str)
def test_layer_norm_on_permuted_views(hk, cuda, dt, case):
    import torch
    stored, perm = case
    vshape = _shape_of_view(stored, perm)
    cols = vshape[-1]
    rows = int(np.prod(vshape[:-1]))
    x = helpers.draw(41, vshape, dtype=dt)
    dy = helpers.draw(42, vshape, dtype=dt)
    g = helpers.draw(43, (cols,), "uniform", 0.5, 1.5, dt)
    b = helpers.draw(44, (cols,), "normal", 0.0, 0.1, dt)
    tg, tb = helpers.to_torch(g, dt, cuda), helpers.to_torch(b, dt, cuda)
    sx, vx = _view(x, perm, dt, cuda)
    assert not vx.is_contiguous() or rows == 1 or min(vshape[:-1]) == 1
    before = sx.clone()
    wy, vy = _out_view(vshape, perm, dt, cuda, pad=16)
    mean, rstd = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.layer_norm_fwd(vx, tg, tb, vy, mean, rstd, 1e-5, stat_kind=1)
    dense_y = torch.empty(vshape, dtype=vx.dtype, device=cuda)
    mean2, rstd2 = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.layer_norm_fwd(vx.contiguous(), tg, tb, dense_y, mean2, rstd2, 1e-5, stat_kind=1)
    torch.cuda.synchronize()
    ey, em, _, ers = oracle.layernorm_fwd(x.reshape(rows, cols), g, b, 1e-5)
    helpers.assert_close(vy.reshape(rows, cols), ey, dt, "y")
    helpers.assert_close(mean, em, "fp32", "mean", scale=1.0)
    helpers.assert_close(rstd, ers, "fp32", "rstd")
    assert torch.equal(vy, dense_y) and torch.equal(mean, mean2) and torch.equal(rstd, rstd2)
    assert torch.equal(sx, before) and _padding_untouched(wy, cols)
    # backward: dy dense, x a permuted view, dx a permuted view of a padded buffer
    tdy = helpers.to_torch(dy, dt, cuda)
    wdx, vdx = _out_view(vshape, perm, dt, cuda, pad=8)
    dg, db = torch.empty_like(tg), torch.empty_like(tb)
    hk.layer_norm_bwd(tdy, vx, tg, None, mean, rstd, vdx, dg, db, 1e-5, stat_kind=1)
    dense_dx = torch.empty(vshape, dtype=vx.dtype, device=cuda)
    dg2, db2 = torch.empty_like(tg), torch.empty_like(tb)
    hk.layer_norm_bwd(tdy, vx.contiguous(), tg, None, mean, rstd, dense_dx, dg2, db2, 1e-5, stat_kind=1)
    torch.cuda.synchronize()
    edx, edg, edb = oracle.layernorm_bwd(dy.reshape(rows, cols), x.reshape(rows, cols), g, helpers.to_numpy(mean),
                                         helpers.to_numpy(rstd))
    helpers.assert_close(vdx.reshape(rows, cols), edx, dt, "dx")
    helpers.assert_close(dg, edg, dt, "dgamma", scale=float(np.sqrt(rows)))
    helpers.assert_close(db, edb, dt, "dbeta", scale=float(np.sqrt(rows)))
    assert torch.equal(vdx, dense_dx)
    assert _padding_untouched(wdx, cols)


@pytest.mark.parametrize("case", VIEWS, ids=str)
def test_rmsnorm_on_permuted_views(hk, cuda, case):
    import torch
    dt = "bf16"
    stored, perm = case
    vshape = _shape_of_view(stored, perm)
    cols = vshape[-1]
    rows = int(np.prod(vshape[:-1]))
    x0 = helpers.draw(51, vshape, dtype=dt)
    res = helpers.draw(52, vshape, dtype=dt)
    w = helpers.draw(53, (cols,), "uniform", 0.8, 1.2, dt)
    dz = helpers.draw(54, vshape, dtype=dt)
    tw = helpers.to_torch(w, dt, cuda)
    _, vx0 = _view(x0, perm, dt, cuda, pad=8)
    tres = helpers.to_torch(res, dt, cuda)                 # dense next to a permuted operand
    wz, vz = _out_view(vshape, perm, dt, cuda, pad=8)
    wxo, vxo = _out_view(vshape, perm, dt, cuda)
    mu, rs = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.dropout_add_ln_fwd(vx0, tres, tw, None, vz, vxo, mu, rs, 1e-6, True)
    torch.cuda.synchronize()
    ez, ex, _, ers = oracle.dropout_add_ln_fwd(x0.reshape(rows, cols), res.reshape(rows, cols), w, None, 1e-6, True)
    helpers.assert_close(vz.reshape(rows, cols), ez, dt, "z")
    helpers.assert_close(vxo.reshape(rows, cols), ex, dt, "x")
    helpers.assert_close(rs, ers, "fp32", "rsigma")
    assert _padding_untouched(wz, cols)
    # backward with the residual stream's gradient coming in (dense) and going out (permuted)
    _, vdz = _view(dz, perm, dt, cuda)
    dxin = helpers.draw(55, vshape, dtype=dt)
    tdxin = helpers.to_torch(dxin, dt, cuda)
    wdx0, vdx0 = _out_view(vshape, perm, dt, cuda, pad=16)
    tdr = torch.empty(vshape, dtype=vdz.dtype, device=cuda)
    dg, db = torch.empty_like(tw), torch.empty_like(tw)
    xsum = helpers.to_numpy(vxo).reshape(rows, cols)
    hk.dropout_add_ln_bwd(vdz, tdxin, vxo, mu, rs, tw, vdx0, tdr, dg, db, True)
    torch.cuda.synchronize()
    edx, edg, _ = oracle.dropout_add_ln_bwd(dz.reshape(rows, cols), dxin.reshape(rows, cols), xsum, helpers.to_numpy(mu),
                                            helpers.to_numpy(rs), w, True)
    helpers.assert_close(vdx0.reshape(rows, cols), edx, dt, "dx0")
    assert torch.equal(vdx0, tdr)
    helpers.assert_close(dg, edg, dt, "dgamma", scale=float(np.sqrt(rows)))
    assert _padding_untouched(wdx0, cols)
    # the plain backward of an RMSNorm layer on the same views: dx and dgamma only, no residual stream (the lean
    # instances, with a running walk index where the rows lie on several levels)
    wdx1, vdx1 = _out_view(vshape, perm, dt, cuda, pad=16)
    dg1 = torch.empty_like(tw)
    hk.dropout_add_ln_bwd(vdz, None, vxo, mu, rs, tw, vdx1, None, dg1, None, True)
    torch.cuda.synchronize()
    edx1, edg1, _ = oracle.dropout_add_ln_bwd(dz.reshape(rows, cols), None, xsum, helpers.to_numpy(mu),
                                              helpers.to_numpy(rs), w, True)
    helpers.assert_close(vdx1.reshape(rows, cols), edx1, dt, "dx0")
    helpers.assert_close(dg1, edg1, dt, "dgamma", scale=float(np.sqrt(rows)))
    assert _padding_untouched(wdx1, cols)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("case", VIEWS, ids=str)
def test_softmax_on_permuted_views(hk, cuda, dt, case):
    import torch
    stored, perm = case
    vshape = _shape_of_view(stored, perm)
    cols = vshape[-1]
    rows = int(np.prod(vshape[:-1]))
    x = helpers.draw(61, vshape, "normal", 0.0, 3.0, dt)
    dy = helpers.draw(62, vshape, dtype=dt)
    sx, vx = _view(x, perm, dt, cuda)
    before = sx.clone()
    wy, vy = _out_view(vshape, perm, dt, cuda, pad=8)
    hk.softmax_fwd(vx, vy)
    dense = torch.empty(vshape, dtype=vx.dtype, device=cuda)
    hk.softmax_fwd(vx.contiguous(), dense)
    torch.cuda.synchronize()
    helpers.assert_close(vy.reshape(rows, cols), oracle.softmax_fwd(x.reshape(rows, cols)), dt, "softmax")
    assert torch.equal(vy, dense) and torch.equal(sx, before) and _padding_untouched(wy, cols)
    y = helpers.to_numpy(vy).reshape(rows, cols)
    _, vdy = _view(dy, perm, dt, cuda, pad=16)
    tdx = torch.empty(vshape, dtype=vx.dtype, device=cuda)       # dense output next to permuted inputs
    hk.softmax_bwd(vy, vdy, tdx)
    torch.cuda.synchronize()
    helpers.assert_close(tdx.reshape(rows, cols), oracle.softmax_bwd(y, dy.reshape(rows, cols)), dt, "softmax gradient",
                         ordinary_rtol=helpers.SOFTMAX_GRADIENT_ORDINARY_RTOL,
                         strict_rtol=helpers.SOFTMAX_GRADIENT_STRICT_RTOL if dt == "fp32" else None)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("case", [((2, 3, 5, 1000), (0, 2, 1)), ((4, 6, 32000), (1, 0)), ((3, 2, 2, 264), (2, 1, 0))], ids=str)
def test_sparse_cross_entropy_on_permuted_views(hk, cuda, dt, case):
    import torch
    stored, perm = case
    vshape = _shape_of_view(stored, perm)
    cols = vshape[-1]
    rows = int(np.prod(vshape[:-1]))
    x = helpers.draw(71, vshape, "normal", 0.0, 2.0, dt)
    rng = np.random.default_rng(72)
    lab = rng.integers(0, cols, rows).astype(np.int64)
    lab[rng.random(rows) < 0.2] = -100
    gl = helpers.draw(73, (rows,), dtype=dt)
    sx, vx = _view(x, perm, dt, cuda)
    tl = torch.from_numpy(lab).to(cuda)
    loss = torch.empty(rows, dtype=vx.dtype, device=cuda)
    hk.sce_sparse_fwd(vx, tl, loss, -100)
    loss2 = torch.empty_like(loss)
    hk.sce_sparse_fwd(vx.contiguous(), tl, loss2, -100)
    torch.cuda.synchronize()
    helpers.assert_close(loss, oracle.sce_sparse_fwd(x.reshape(rows, cols), lab, -100), dt, "loss")
    assert torch.equal(loss, loss2)
    assert bool((loss[tl == -100].float() == 0).all())
    wd, vd = _out_view(vshape, perm, dt, cuda, pad=8)
    tgl = helpers.to_torch(gl, dt, cuda)
    hk.sce_sparse_bwd(vx, tl, tgl, vd, -100)
    dense = torch.empty(vshape, dtype=vx.dtype, device=cuda)
    hk.sce_sparse_bwd(vx.contiguous(), tl, tgl, dense, -100)
    torch.cuda.synchronize()
    helpers.assert_close(vd.reshape(rows, cols), oracle.sce_sparse_bwd(x.reshape(rows, cols), lab, gl, -100), dt, "dlogits")
    assert torch.equal(vd, dense) and _padding_untouched(wd, cols)
    assert bool((vd.reshape(rows, cols)[tl == -100].float() == 0).all())


def test_walk_order_does_not_change_results(hk, cuda):
    """The launch walks the levels by ascending step; a view whose longest level has the smallest step (and one
    whose row count on a level exceeds a grid's y / z range) still gets every row's statistics in the row's own
    number."""
    import torch
    dt = "fp32"
    S, B, D = 70000, 2, 64                       # stored [S, B, D], used as [B, S, D]: level 0 = S rows, 128 apart
    x = helpers.draw(81, (B, S, D), dtype=dt)
    sx, vx = _view(x, (1, 0), dt, cuda)
    g = helpers.draw(82, (D,), "uniform", 0.5, 1.5, dt)
    tg = helpers.to_torch(g, dt, cuda)
    y = torch.empty((B, S, D), device=cuda)
    mean, rstd = torch.empty(B * S, device=cuda), torch.empty(B * S, device=cuda)
    hk.layer_norm_fwd(vx, tg, None, y, mean, rstd, 1e-5, stat_kind=1)
    torch.cuda.synchronize()
    ey, em, _, ers = oracle.layernorm_fwd(x.reshape(B * S, D), g, np.zeros(D), 1e-5)
    helpers.assert_close(y.reshape(B * S, D), ey, dt, "y")
    helpers.assert_close(mean, em, dt, "mean", scale=1.0)
    helpers.assert_close(rstd, ers, dt, "rstd")
