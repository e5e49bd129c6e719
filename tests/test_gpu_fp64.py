"""float64 data goes through the generic kernels of every operator (the reference dispatches its
floating-point kernels on fp64 too): parity with the float64 oracle at 1e-10."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-10


def _draw64(seed, shape, scale=1.0, shift=0.0):
    return helpers.rng(seed).standard_normal(shape) * scale + shift


def test_layer_norm_fp64(hk, cuda):
    import torch
    rows, cols, eps = 19, 1000, 1e-5
    x, dy = _draw64(1, (rows, cols)), _draw64(2, (rows, cols))
    gamma, beta = _draw64(3, (cols,), 0.2, 1.0), _draw64(4, (cols,), 0.1)
    # the oracle takes float32-representable inputs; feed it exactly what the device sees
    x, dy, gamma, beta = (v.astype(np.float32).astype(np.float64) for v in (x, dy, gamma, beta))
    ey, emean, evar, erstd = oracle.layernorm_fwd(x.astype(np.float32), gamma.astype(np.float32), beta.astype(np.float32), eps)
    tx, tg, tb, tdy = (helpers.to_torch(v, "fp64", cuda) for v in (x, gamma, beta, dy))
    ty = torch.empty_like(tx)
    tmean = torch.empty(rows, dtype=torch.float64, device=cuda)
    tvar = torch.empty(rows, dtype=torch.float64, device=cuda)
    hk.layer_norm_fwd(tx, tg, tb, ty, tmean, tvar, eps, stat_kind=0)
    torch.cuda.synchronize()
    helpers.assert_close(ty, ey, "fp64", "y", rtol=TOL)
    helpers.assert_close(tvar, evar, "fp64", "var", rtol=TOL)
    edx, edg, edb = oracle.layernorm_bwd(dy.astype(np.float32), x.astype(np.float32), gamma.astype(np.float32),
                                         emean, erstd)
    tdx, tdg, tdb = torch.empty_like(tx), torch.empty_like(tg), torch.empty_like(tg)
    hk.layer_norm_bwd(tdy, tx, tg, None, tmean, tvar, tdx, tdg, tdb, eps, stat_kind=0)
    torch.cuda.synchronize()
    helpers.assert_close(tdx, edx, "fp64", "dx", rtol=1e-9)
    helpers.assert_close(tdg, edg, "fp64", "dgamma", rtol=1e-9)
    helpers.assert_close(tdb, edb, "fp64", "dbeta", rtol=1e-9)
    with pytest.raises(hk.HkError):     # fp64 data keeps fp64 statistics
        hk.layer_norm_fwd(tx, tg, tb, ty, tmean.float(), tvar.float(), eps, stat_kind=1)
    with pytest.raises(hk.HkError):     # the fused dropout-add-norm has no fp64 variant
        hk.dropout_add_ln_fwd(tx, None, tg, None, ty, None, tmean.float(), tvar.float(), eps, True)


@pytest.mark.parametrize("shape,dim", [((11, 257), -1), ((6, 40, 9), 1)])
def test_softmax_fp64(hk, cuda, shape, dim):
    import torch
    x = _draw64(5, shape, 3.0).astype(np.float32).astype(np.float64)
    dy = _draw64(6, shape).astype(np.float32).astype(np.float64)
    tx, tdy = helpers.to_torch(x, "fp64", cuda), helpers.to_torch(dy, "fp64", cuda)
    ty, tdx = torch.empty_like(tx), torch.empty_like(tx)
    hk.softmax_fwd(tx, ty, dim)
    torch.cuda.synchronize()
    helpers.assert_close(ty, oracle.softmax_fwd(x.astype(np.float32), dim), "fp64", "y", rtol=TOL)
    y = ty.cpu().numpy()
    hk.softmax_bwd(ty, tdy, tdx, dim)
    torch.cuda.synchronize()
    want = y * dy - y * np.sum(y * dy, axis=dim, keepdims=True)
    helpers.assert_close(tdx, want, "fp64", "dx", rtol=1e-9)


def test_cross_entropy_fp64(hk, cuda):
    import torch
    rows, cols, ignored = 37, 501, -100
    x = _draw64(7, (rows, cols), 2.0).astype(np.float32).astype(np.float64)
    labels = helpers.rng(8).integers(0, cols, size=rows).astype(np.int64)
    labels[::6] = ignored
    gl = _draw64(9, (rows,)).astype(np.float32).astype(np.float64)
    tx, tgl = helpers.to_torch(x, "fp64", cuda), helpers.to_torch(gl, "fp64", cuda)
    tl = torch.from_numpy(labels).to(cuda)
    tloss = torch.empty(rows, dtype=torch.float64, device=cuda)
    tgrad = torch.empty_like(tx)
    hk.sce_sparse_fwd(tx, tl, tloss, ignored)
    hk.sce_sparse_bwd(tx, tl, tgl, tgrad, ignored)
    torch.cuda.synchronize()
    helpers.assert_close(tloss, oracle.sce_sparse_fwd(x.astype(np.float32), labels, ignored), "fp64", "loss", rtol=TOL)
    helpers.assert_close(tgrad, oracle.sce_sparse_bwd(x.astype(np.float32), labels, gl.astype(np.float32), ignored),
                         "fp64", "grad", rtol=1e-9)
    assert np.all(tloss.cpu().numpy()[labels == ignored] == 0.0)
    lab = helpers.rng(10).random((rows, cols))
    lab = (lab / lab.sum(1, keepdims=True)).astype(np.float32).astype(np.float64)
    tlab = helpers.to_torch(lab, "fp64", cuda)
    hk.sce_dense_fwd(tx, tlab, tloss)
    hk.sce_dense_bwd(tx, tlab, tgl, tgrad)
    torch.cuda.synchronize()
    helpers.assert_close(tloss, oracle.sce_dense_fwd(x.astype(np.float32), lab.astype(np.float32)), "fp64", "dense loss", rtol=TOL)
    helpers.assert_close(tgrad, oracle.sce_dense_bwd(x.astype(np.float32), lab.astype(np.float32), gl.astype(np.float32)),
                         "fp64", "dense grad", rtol=1e-9)
