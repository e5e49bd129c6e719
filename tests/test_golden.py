"""Golden fixtures (tests/golden/rowwise_small.npz, written by make_golden.py from
the CPU oracle): the oracle must keep reproducing them, and the GPU kernels must
match them through the C-ABI."""
import os

import numpy as np
import pytest

import helpers
import oracle

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rowwise_small.npz"))


def g(dt, k):
    return G["%s/%s" % (dt, k)]


@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_oracle_reproduces_golden(dt):
    x, gamma, beta, dy = g(dt, "x"), g(dt, "gamma"), g(dt, "beta"), g(dt, "dy")
    y, mean, var, rstd = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
    assert np.array_equal(y, g(dt, "ln_y")) and np.array_equal(var, g(dt, "ln_var"))
    z, _, mu, rs = oracle.dropout_add_ln_fwd(x, None, gamma, None, 1e-6, True)
    assert np.array_equal(z, g(dt, "rms_z")) and np.array_equal(rs, g(dt, "rms_rs"))
    assert np.array_equal(oracle.softmax_fwd(g(dt, "sm_x")), g(dt, "sm_y"))
    assert np.array_equal(oracle.sce_sparse_fwd(x, g(dt, "labels"), -100), g(dt, "sce_loss"))
    assert np.array_equal(oracle.reduce(g(dt, "sm_x"), [0, 1], "sum"), g(dt, "red_sum01"))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_gpu_matches_golden(hk, cuda, dt):
    import torch
    T = lambda k, d=dt: helpers.to_torch(g(dt, k), d, cuda)
    x, gamma, beta, dy = T("x"), T("gamma"), T("beta"), T("dy")
    rows, cols = x.shape
    y = torch.empty_like(x); mean = torch.empty(rows, device=cuda); rstd = torch.empty(rows, device=cuda)
    hk.layer_norm_fwd(x, gamma, beta, y, mean, rstd, 1e-5, stat_kind=1)
    dx = torch.empty_like(x); dg = torch.empty_like(gamma); db = torch.empty_like(gamma)
    hk.layer_norm_bwd(dy, x, gamma, beta, T("ln_mean", "fp32"), T("ln_rstd", "fp32"), dx, dg, db, 1e-5,
                      stat_kind=1, clamp_gamma=True)
    z = torch.empty_like(x); mu = torch.empty(rows, device=cuda); rs = torch.empty(rows, device=cuda)
    hk.dropout_add_ln_fwd(x, None, gamma, None, z, None, mu, rs, 1e-6, True)
    rdx = torch.empty_like(x); rdg = torch.empty_like(gamma); rdb = torch.empty_like(gamma)
    hk.dropout_add_ln_bwd(dy, None, x, T("rms_mu", "fp32"), T("rms_rs", "fp32"), gamma, rdx, None, rdg, rdb, True)
    sx, sdy = T("sm_x"), T("sm_dy")
    sy = torch.empty_like(sx); sdx = torch.empty_like(sx)
    hk.softmax_fwd(sx, sy)
    hk.softmax_bwd(helpers.to_torch(oracle.round_to(g(dt, "sm_y"), dt), dt, cuda), sdy, sdx)
    lab = torch.from_numpy(g(dt, "labels")).to(cuda)
    loss = torch.empty(rows, dtype=x.dtype, device=cuda); dlog = torch.empty_like(x)
    hk.sce_sparse_fwd(x, lab, loss, -100)
    hk.sce_sparse_bwd(x, lab, T("grad_loss"), dlog, -100)
    r0 = torch.empty(24, dtype=x.dtype, device=cuda); r1 = torch.empty((4, 3), dtype=x.dtype, device=cuda)
    hk.reduce(sx, r0, [0, 1], "sum"); hk.reduce(sx, r1, [2], "mean")
    torch.cuda.synchronize()
    for got, key, kw in ((y, "ln_y", {}), (rstd, "ln_rstd", {"dtype": "fp32"}), (dx, "ln_dx", {}), (dg, "ln_dgamma", {}),
                         (db, "ln_dbeta", {}), (z, "rms_z", {}), (rs, "rms_rs", {"dtype": "fp32"}), (rdx, "rms_dx", {}),
                         (rdg, "rms_dgamma", {}), (sy, "sm_y", {}), (sdx, "sm_dx", {}), (loss, "sce_loss", {}),
                         (dlog, "sce_dlogits", {}), (r0, "red_sum01", {}), (r1, "red_mean2", {})):
        helpers.assert_close(got, g(dt, key), kw.get("dtype", dt), key)
    assert torch.count_nonzero(dlog[[1, 5]]) == 0 and torch.count_nonzero(loss[[1, 5]]) == 0
