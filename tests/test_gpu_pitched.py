"""Row-pitched operands: inputs and outputs that are column slices `w[:, a:a + cols]` of wider buffers go through
the *_pitched entry points as they are, without a dense copy.  Every result is compared with the oracle and,
bit for bit, with the same call on dense copies; what lies outside the output slice must stay untouched.
Pitches that are a whole number of 16-byte vectors take the 128-bit kernels, odd pitches and offsets the
element-wise fallbacks."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

# (rows, cols, pitch, column offset): vector path (pitch and offset multiples of 8), then the fallbacks
LAYOUTS = [(64, 1024, 1536, 256), (33, 4096, 4104, 8), (300, 264, 520, 0), (5, 5120, 5120 + 64, 64),
           (40, 1000, 1003, 3), (17, 512, 777, 5), (1, 2048, 4096, 1024)]
SENTINEL = 12288.0          # exactly representable in bf16


def _wide(values, pitch, off, dt, dev):
    """A [rows, pitch] tensor filled with the sentinel, `values` in columns [off, off + cols); returns the slice."""
    import torch
    rows, cols = values.shape
    w = torch.full((rows, pitch), SENTINEL, dtype=helpers.load_package().torch_dtype(dt), device=dev)
    w[:, off:off + cols] = helpers.to_torch(values, dt, dev)
    return w, w[:, off:off + cols]


def _out(rows, cols, pitch, off, dt, dev):
    import torch
    w = torch.full((rows, pitch), SENTINEL, dtype=helpers.load_package().torch_dtype(dt), device=dev)
    return w, w[:, off:off + cols]


def _untouched(w, off, cols):
    import torch
    mask = torch.ones(w.shape[1], dtype=torch.bool, device=w.device)
    mask[off:off + cols] = False
    return bool((w[:, mask].float() == SENTINEL).all())


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("layout", LAYOUTS, ids=str)
def test_layer_norm_on_slices(hk, cuda, dt, layout):
    import torch
    rows, cols, pitch, off = layout
    x = helpers.draw(11, (rows, cols), dtype=dt)
    g = helpers.draw(12, (cols,), "uniform", 0.5, 1.5, dt)
    b = helpers.draw(13, (cols,), "normal", 0.0, 0.1, dt)
    dy = helpers.draw(14, (rows, cols), dtype=dt)
    tg, tb = helpers.to_torch(g, dt, cuda), helpers.to_torch(b, dt, cuda)
    _, sx = _wide(x, pitch, off, dt, cuda)
    _, sdy = _wide(dy, pitch + 8, off, dt, cuda)
    wy, sy = _out(rows, cols, pitch + 16, off, dt, cuda)
    mean, rstd = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.layer_norm_fwd(sx, tg, tb, sy, mean, rstd, 1e-5, stat_kind=1)
    dense_y = torch.empty(rows, cols, dtype=sx.dtype, device=cuda)
    mean2, rstd2 = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.layer_norm_fwd(sx.contiguous(), tg, tb, dense_y, mean2, rstd2, 1e-5, stat_kind=1)
    torch.cuda.synchronize()
    ey, em, _, ers = oracle.layernorm_fwd(x, g, b, 1e-5)
    helpers.assert_close(sy, ey, dt, "y")
    helpers.assert_close(rstd, ers, "fp32", "rstd")
    if pitch % 8 == 0 and off % 8 == 0:          # same kernel, same arithmetic: the same bits
        assert torch.equal(sy, dense_y) and torch.equal(mean, mean2) and torch.equal(rstd, rstd2)
    assert _untouched(wy, off, cols)
    # backward: pitched dy, x and dx
    wdx, sdx = _out(rows, cols, pitch + 24, off, dt, cuda)
    dg, db = torch.empty_like(tg), torch.empty_like(tb)
    hk.layer_norm_bwd(sdy, sx, tg, None, mean, rstd, sdx, dg, db, 1e-5, stat_kind=1)
    torch.cuda.synchronize()
    edx, edg, edb = oracle.layernorm_bwd(dy, x, g, helpers.to_numpy(mean), helpers.to_numpy(rstd))
    helpers.assert_close(sdx, edx, dt, "dx")
    helpers.assert_close(dg, edg, dt, "dgamma", scale=float(np.sqrt(rows)))
    helpers.assert_close(db, edb, dt, "dbeta", scale=float(np.sqrt(rows)))
    assert _untouched(wdx, off, cols)


@pytest.mark.parametrize("layout", LAYOUTS[:5], ids=str)
def test_rmsnorm_with_residual_on_slices(hk, cuda, layout):
    import torch
    dt = "bf16"
    rows, cols, pitch, off = layout
    x0 = helpers.draw(21, (rows, cols), dtype=dt)
    res = helpers.draw(22, (rows, cols), dtype=dt)
    w = helpers.draw(23, (cols,), "uniform", 0.8, 1.2, dt)
    dz = helpers.draw(24, (rows, cols), dtype=dt)
    tw = helpers.to_torch(w, dt, cuda)
    _, sx0 = _wide(x0, pitch, off, dt, cuda)
    _, sres = _wide(res, pitch + 8, off, dt, cuda)
    wz, sz = _out(rows, cols, pitch, off, dt, cuda)
    wx, sxo = _out(rows, cols, pitch + 16, off, dt, cuda)
    mu, rs = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    hk.dropout_add_ln_fwd(sx0, sres, tw, None, sz, sxo, mu, rs, 1e-6, True)
    torch.cuda.synchronize()
    ez, ex, _, ers = oracle.dropout_add_ln_fwd(x0, res, w, None, 1e-6, True)
    helpers.assert_close(sz, ez, dt, "z")
    helpers.assert_close(sxo, ex, dt, "x")
    helpers.assert_close(rs, ers, "fp32", "rsigma")
    assert _untouched(wz, off, cols) and _untouched(wx, off, cols)
    # backward with a gradient of the residual stream coming in and going out, all on slices
    _, sdz = _wide(dz, pitch + 8, off, dt, cuda)
    dxin = helpers.draw(25, (rows, cols), dtype=dt)
    _, sdxin = _wide(dxin, pitch, off, dt, cuda)
    wdx0, sdx0 = _out(rows, cols, pitch + 8, off, dt, cuda)
    wdr, sdr = _out(rows, cols, pitch, off, dt, cuda)
    dg, db = torch.empty_like(tw), torch.empty_like(tw)
    xsum = helpers.to_numpy(sxo)
    hk.dropout_add_ln_bwd(sdz, sdxin, sxo, mu, rs, tw, sdx0, sdr, dg, db, True)
    torch.cuda.synchronize()
    edx, edg, _ = oracle.dropout_add_ln_bwd(dz, dxin, xsum, helpers.to_numpy(mu), helpers.to_numpy(rs), w, True)
    helpers.assert_close(sdx0, edx, dt, "dx0")
    assert torch.equal(sdx0, sdr)
    helpers.assert_close(dg, edg, dt, "dgamma", scale=float(np.sqrt(rows)))
    assert _untouched(wdx0, off, cols) and _untouched(wdr, off, cols)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("layout", LAYOUTS, ids=str)
def test_softmax_on_slices(hk, cuda, dt, layout):
    import torch
    rows, cols, pitch, off = layout
    x = helpers.draw(31, (rows, cols), "normal", 0.0, 3.0, dt)
    dy = helpers.draw(32, (rows, cols), dtype=dt)
    _, sx = _wide(x, pitch, off, dt, cuda)
    wy, sy = _out(rows, cols, pitch + 8, off, dt, cuda)
    hk.softmax_fwd(sx, sy)
    dense = torch.empty(rows, cols, dtype=sx.dtype, device=cuda)
    hk.softmax_fwd(sx.contiguous(), dense)
    torch.cuda.synchronize()
    helpers.assert_close(sy, oracle.softmax_fwd(x), dt, "softmax")
    if pitch % 8 == 0 and off % 8 == 0:
        assert torch.equal(sy, dense)
    assert _untouched(wy, off, cols)
    y = helpers.to_numpy(sy)
    _, sdy = _wide(dy, pitch + 16, off, dt, cuda)
    wdx, sdx = _out(rows, cols, pitch, off, dt, cuda)
    hk.softmax_bwd(sy, sdy, sdx)
    torch.cuda.synchronize()
    helpers.assert_close(sdx, oracle.softmax_bwd(y, dy), dt, "softmax gradient",
                         ordinary_rtol=helpers.SOFTMAX_GRADIENT_ORDINARY_RTOL,
                         strict_rtol=helpers.SOFTMAX_GRADIENT_STRICT_RTOL if dt == "fp32" else None)
    assert _untouched(wdx, off, cols)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("layout", [(48, 32000, 32768, 0), (48, 1000, 1024, 16), (9, 777, 1001, 7)], ids=str)
def test_cross_entropy_on_a_padded_vocabulary(hk, cuda, dt, layout):
    """Logits whose rows are padded (a vocabulary rounded up for the tensor-parallel split): the loss and its
    gradient over the real columns only."""
    import torch
    rows, cols, pitch, off = layout
    x = helpers.draw(41, (rows, cols), "normal", 0.0, 2.0, dt)
    lab = helpers.rng(42).integers(0, cols, rows).astype(np.int64)
    lab[::5] = -100
    tl = torch.from_numpy(lab).to(cuda)
    _, sx = _wide(x, pitch, off, dt, cuda)
    loss = torch.empty(rows, dtype=sx.dtype, device=cuda)
    hk.sce_sparse_fwd(sx, tl, loss, -100)
    dense_loss = torch.empty_like(loss)
    hk.sce_sparse_fwd(sx.contiguous(), tl, dense_loss, -100)
    torch.cuda.synchronize()
    helpers.assert_close(loss, oracle.sce_sparse_fwd(x, lab, -100), dt, "loss")
    if pitch % 8 == 0 and off % 8 == 0:
        assert torch.equal(loss, dense_loss)
    gl = helpers.draw(43, (rows,), "uniform", 0.5, 1.5, dt)
    tgl = helpers.to_torch(gl, dt, cuda)
    wdx, sdx = _out(rows, cols, pitch + 8, off, dt, cuda)
    hk.sce_sparse_bwd(sx, tl, tgl, sdx, -100)
    torch.cuda.synchronize()
    edx = oracle.sce_sparse_bwd(x, lab, gl, -100)
    helpers.assert_close(sdx, edx, dt, "dlogits")
    assert not sdx[::5].float().any()            # ignored rows are zero rows inside the slice ...
    assert _untouched(wdx, off, cols)            # ... and nothing is written outside it


def test_pitch_arguments_are_checked(hk, cuda):
    import ctypes
    import torch
    x = torch.zeros(4, 64, device=cuda)
    st = torch.zeros(4, device=cuda)
    lib = hk.lib()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.hk_layer_norm_fwd_pitched(6, p(x), ctypes.c_int64(32), None, None, p(x), ctypes.c_int64(64), p(st), p(st), 6, 1,
                                       ctypes.c_int64(4), ctypes.c_int64(64), ctypes.c_float(1e-5), None)
    assert rc == -1 and b"pitch" in lib.hk_last_error()      # a pitch below the row length
    rc = lib.hk_softmax_fwd_pitched(6, p(x), ctypes.c_int64(64), p(x), ctypes.c_int64(0), ctypes.c_int64(4),
                                    ctypes.c_int64(64), None)
    assert rc == -1
    with pytest.raises(hk.HkError):
        hk.softmax_fwd(x.t(), torch.empty(64, 4, device=cuda))   # a transposed view has no unit-stride last dimension
