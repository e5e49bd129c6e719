"""GPU parity of spatial batch normalisation in training mode (hk_batch_norm_fwd / _bwd) against the oracle's
restatement of cuDNN's documented arithmetic: outputs, saved and running statistics, all three gradients."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

SHAPES = [(8, 16, 14, 14), (2, 3, 5, 7), (32, 64, 8, 8), (1, 4, 1, 1), (4, 7, 33, 1), (64, 256, 4, 4), (3, 5, 9)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16", "fp64"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_forward_and_backward(hk, cuda, dtype, shape):
    import torch
    g = helpers.rng(sum(shape))
    C = shape[1]
    pt = "fp64" if dtype == "fp64" else "fp32"             # parameters and statistics: fp32 for 16-bit data
    rnd = lambda a, d: a.astype(np.float64) if d == "fp64" else oracle.round_to(a.astype(np.float32), d)
    x = rnd(g.standard_normal(shape) * 2 + 3, dtype)       # a mean well away from zero
    scale = rnd(g.uniform(0.5, 1.5, C), pt); bias = rnd(g.standard_normal(C), pt)
    rm = rnd(g.standard_normal(C), pt); rv = rnd(g.uniform(0.5, 2.0, C), pt)
    dy = rnd(g.standard_normal(shape), dtype)
    momentum, eps = 0.1, 1e-5
    ey, erm, erv, emean, einv = oracle.batch_norm_fwd(x, scale, bias, rm, rv, momentum, eps)
    tx = helpers.to_torch(x, dtype, cuda); ts = helpers.to_torch(scale, pt, cuda); tb = helpers.to_torch(bias, pt, cuda)
    trm = helpers.to_torch(rm, pt, cuda); trv = helpers.to_torch(rv, pt, cuda)
    ty = torch.empty_like(tx); smean = torch.empty_like(ts); sinv = torch.empty_like(ts)
    hk.batch_norm_fwd(tx, ts, tb, ty, momentum, eps, trm, trv, smean, sinv)
    torch.cuda.synchronize()
    m = x.size // C
    helpers.assert_close(ty, ey, dtype, "y")
    helpers.assert_close(smean, emean, pt, "save_mean", scale=float(np.sqrt(np.mean(x.astype(np.float64) ** 2))))
    if m > 1:
        helpers.assert_close(sinv, einv, pt, "save_invstd", rtol=1e-4 if pt == "fp32" else None)
        helpers.assert_close(trv, erv, pt, "running_var", rtol=1e-4 if pt == "fp32" else None)
    helpers.assert_close(trm, erm, pt, "running_mean", scale=1.0)
    # backward from the statistics as saved
    sm = helpers.to_numpy(smean).astype(np.float64); si = helpers.to_numpy(sinv).astype(np.float64)
    edx, eds, edb = oracle.batch_norm_bwd(dy, x, scale, sm, si)
    tdy = helpers.to_torch(dy, dtype, cuda)
    dx = torch.empty_like(tx); ds = torch.empty_like(ts); db = torch.empty_like(ts)
    hk.batch_norm_bwd(tdy, tx, ts, dx, ds, db, smean, sinv)
    torch.cuda.synchronize()
    helpers.assert_close(dx, edx, dtype, "dx", rtol=2e-2 if dtype in ("bf16", "fp16") else (1e-4 if dtype == "fp32" else None))
    helpers.assert_close(ds, eds, pt, "dscale", rtol=1e-4 if pt == "fp32" else None)
    helpers.assert_close(db, edb, pt, "dbias", rtol=1e-4 if pt == "fp32" else None)


def test_properties_at_size(hk, cuda):
    """[128, 256, 28, 28] bf16: per channel the output has mean bias and variance scale^2 var / (var + eps);
    the gradient of x sums to zero over every channel."""
    import torch
    N, C, H, W = 128, 256, 28, 28
    x = (torch.randn(N, C, H, W, device=cuda) * 1.5 + 0.5).bfloat16()
    scale = torch.rand(C, device=cuda) + 0.5; bias = torch.randn(C, device=cuda)
    y = torch.empty_like(x); sm = torch.empty(C, device=cuda); si = torch.empty(C, device=cuda)
    hk.batch_norm_fwd(x, scale, bias, y, 0.1, 1e-5, None, None, sm, si)
    torch.cuda.synchronize()
    yf = y.float()
    assert torch.allclose(yf.mean(dim=(0, 2, 3)), bias, atol=2e-2)
    assert torch.allclose(yf.var(dim=(0, 2, 3), unbiased=False), scale ** 2, rtol=3e-2)
    assert torch.allclose(sm, x.float().mean(dim=(0, 2, 3)), atol=1e-4)
    dy = torch.randn_like(yf).bfloat16()
    dx = torch.empty_like(x); ds = torch.empty(C, device=cuda); db = torch.empty(C, device=cuda)
    hk.batch_norm_bwd(dy, x, scale, dx, ds, db, sm, si)
    torch.cuda.synchronize()
    assert torch.allclose(db, dy.float().sum(dim=(0, 2, 3)), rtol=1e-4, atol=1e-2)
    per_channel = dx.float().sum(dim=(0, 2, 3)).abs()
    assert float(per_channel.max()) < 2e-2 * float(dx.float().abs().sum(dim=(0, 2, 3)).max())


def test_refused_and_empty(hk, cuda):
    import torch
    x = torch.zeros(2, 3, 4, 4, device=cuda)
    p = torch.ones(3, device=cuda)
    with pytest.raises(hk.HkError) as e:
        hk.batch_norm_fwd(x.long(), p, p, x.long(), 0.1, 1e-5, None, None, None, None)
    assert e.value.code == -2
    import ctypes
    rc = hk.lib().hk_batch_norm_fwd(6, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(p.data_ptr()),
                                    ctypes.c_void_p(p.data_ptr()), ctypes.c_void_p(x.data_ptr()), ctypes.c_double(0.1),
                                    ctypes.c_double(1e-5), None, None, None, None, ctypes.c_int64(2),
                                    ctypes.c_int64(3), ctypes.c_int64(16), None, ctypes.c_size_t(0), None)
    assert rc == -4                                       # no workspace
    e0 = torch.empty(0, 3, 4, 4, device=cuda)
    hk.batch_norm_fwd(e0, p, p, e0.clone(), 0.1, 1e-5, None, None, None, None)
    c0 = torch.empty(2, 0, 4, 4, device=cuda)             # no channel at all: nothing to do, forward and backward
    hk.batch_norm_fwd(c0, p[:0], p[:0], c0.clone(), 0.1, 1e-5, None, None, None, None)
    hk.batch_norm_bwd(c0, c0, p[:0], c0.clone(), p[:0].clone(), p[:0].clone(), p[:0], p[:0])
    # a constant channel: variance 0, output = bias, finite statistics
    c = torch.full((4, 2, 8, 8), 3.0, device=cuda)
    y = torch.empty_like(c); sm = torch.empty(2, device=cuda); si = torch.empty(2, device=cuda)
    hk.batch_norm_fwd(c, torch.ones(2, device=cuda), torch.full((2,), 0.25, device=cuda), y, 0.1, 1e-5, None, None, sm, si)
    torch.cuda.synchronize()
    assert (y == 0.25).all() and (sm == 3.0).all() and torch.allclose(si, torch.full((2,), 1e-5 ** -0.5, device=cuda))


@pytest.mark.parametrize("shape", [(0, 8, 4, 4), (4, 0, 4, 4), (4, 8, 0, 4)])
def test_batch_norm_empty_shapes(hk, cuda, shape):
    """An array without elements (no samples, no channels, no pixels) returns at once, forward and backward, and
    needs no workspace; running statistics are left as they are."""
    import torch
    N, C = shape[0], shape[1]
    x = torch.empty(shape, dtype=torch.float32, device=cuda)
    y = torch.empty_like(x)
    scale = torch.ones(C, device=cuda); bias = torch.zeros(C, device=cuda)
    rm = torch.full((C,), 3.0, device=cuda); rv = torch.full((C,), 5.0, device=cuda)
    sm = torch.empty(C, device=cuda); si = torch.empty(C, device=cuda)
    assert hk.batch_norm_workspace_bytes(x) == 0
    hk.batch_norm_fwd(x, scale, bias, y, 0.1, 1e-5, rm, rv, sm, si)
    dx = torch.empty_like(x); ds = torch.empty(C, device=cuda); db = torch.empty(C, device=cuda)
    hk.batch_norm_bwd(y, x, scale, dx, ds, db, sm, si)
    torch.cuda.synchronize()
    assert bool((rm == 3.0).all()) and bool((rv == 5.0).all())
