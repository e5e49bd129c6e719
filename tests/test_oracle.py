"""Pins the CPU oracle (oracle/oracle.c) without the GPU: closed forms and
invariants, brute force in pure Python on tiny inputs, finite differences for
every backward, and cross-checks against an independent library (torch CPU in
float64).  The reference repository has no tests or golden vectors for these
kernels, so these checks are what anchors the oracle."""
import math

import numpy as np
import pytest
import torch

import helpers
import oracle

F64 = dict(rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------------------
# bf16 conversion (hetu/core/bfloat16.h:41-53)
# ---------------------------------------------------------------------------
def test_bf16_roundtrip_is_exhaustive():
    bits = np.arange(1 << 16, dtype=np.uint16)
    f = oracle.bf16_bits_to_f32(bits)
    back = oracle.f32_to_bf16_bits(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])           # every non-NaN pattern survives
    assert np.all(back[nan] == 0x7FC0)                      # NaN canonicalises to 0x7FC0
    # agrees with torch's round-to-nearest-even conversion on random floats
    g = np.random.default_rng(0).standard_normal(200000).astype(np.float32) * 1e3
    t = torch.from_numpy(g).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(g), t)


def test_bf16_ties_round_to_even():
    def f(u):
        return np.array([u], dtype=np.uint32).view(np.float32)
    assert oracle.f32_to_bf16_bits(f(0x3F808000))[0] == 0x3F80   # tie, even stays
    assert oracle.f32_to_bf16_bits(f(0x3F818000))[0] == 0x3F82   # tie, odd rounds up
    assert oracle.f32_to_bf16_bits(f(0x3F808001))[0] == 0x3F81   # above the tie
    assert oracle.f32_to_bf16_bits(f(0x7F7FFFFF))[0] == 0x7F80   # max float rounds to inf


# ---------------------------------------------------------------------------
# LayerNorm
# ---------------------------------------------------------------------------
def _ln_inputs(rows=5, cols=24, seed=0):
    g = np.random.default_rng(seed)
    return (g.standard_normal((rows, cols)).astype(np.float32), (g.random(cols) + 0.5).astype(np.float32),
            (g.standard_normal(cols) * 0.1).astype(np.float32), g.standard_normal((rows, cols)).astype(np.float32))


def test_layernorm_fwd_brute_force_and_invariants():
    x, gamma, beta, _ = _ln_inputs(3, 8)
    eps = 1e-5
    y, mean, var, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    for r in range(3):                                       # plain Python, textbook formula
        row = [float(v) for v in x[r]]
        mu = sum(row) / 8
        v = sum((a - mu) ** 2 for a in row) / 8
        assert math.isclose(mean[r], mu, rel_tol=1e-12, abs_tol=1e-15) and math.isclose(var[r], v, rel_tol=1e-12)
        for c in range(8):
            want = (row[c] - mu) / math.sqrt(v + eps) * float(gamma[c]) + float(beta[c])
            assert math.isclose(y[r, c], want, rel_tol=1e-12, abs_tol=1e-14)
    xhat = (y - beta) / gamma
    assert np.allclose(xhat.mean(1), 0, atol=1e-12)
    assert np.allclose((xhat ** 2).mean(1), var / (var + eps), **F64)
    assert np.allclose(rstd, 1 / np.sqrt(var + eps), **F64)
    # a constant row: var = 0 (never negative), y = beta
    yc, _, vc, _ = oracle.layernorm_fwd(np.full((2, 8), 7.5, np.float32), gamma, beta, eps)
    assert np.all(vc == 0) and np.allclose(yc, beta.astype(np.float64)[None, :], atol=0)


def test_layernorm_matches_torch_float64():
    x, gamma, beta, dy = _ln_inputs(7, 40, 1)
    eps = 1e-5
    y, mean, var, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tg = torch.tensor(gamma, dtype=torch.float64, requires_grad=True)
    tb = torch.tensor(beta, dtype=torch.float64, requires_grad=True)
    ty = torch.nn.functional.layer_norm(tx, (40,), tg, tb, eps)
    assert np.allclose(y, ty.detach().numpy(), **F64)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    dx, dg, db = oracle.layernorm_bwd(dy, x, gamma, mean, rstd)
    assert np.allclose(dx, tx.grad.numpy(), **F64)
    assert np.allclose(dg, tg.grad.numpy(), **F64)
    assert np.allclose(db, tb.grad.numpy(), **F64)
    assert np.allclose(dx.sum(1), 0, atol=1e-12)             # per-row identity
    assert np.allclose(db, dy.astype(np.float64).sum(0), **F64)


def test_layernorm_bwd_finite_differences():
    x, gamma, beta, dy = _ln_inputs(2, 6, 2)
    eps = 1e-3
    _, mean, _, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    dx, dg, db = oracle.layernorm_bwd(dy, x, gamma, mean, rstd)
    h = 1e-3                                                  # inputs are float32: use exactly representable steps

    def loss(xx, gg, bb):
        return float((oracle.layernorm_fwd(xx, gg, bb, eps)[0] * dy).sum())
    for (r, c) in [(0, 0), (1, 3), (0, 5)]:
        xp, xm = x.copy(), x.copy()
        xp[r, c] += np.float32(h); xm[r, c] -= np.float32(h)
        num = (loss(xp, gamma, beta) - loss(xm, gamma, beta)) / float(np.float64(xp[r, c]) - np.float64(xm[r, c]))
        assert math.isclose(num, dx[r, c], rel_tol=2e-4, abs_tol=2e-5)
    for c in (0, 4):
        gp, gm_ = gamma.copy(), gamma.copy()
        gp[c] += np.float32(h); gm_[c] -= np.float32(h)
        num = (loss(x, gp, beta) - loss(x, gm_, beta)) / float(np.float64(gp[c]) - np.float64(gm_[c]))
        assert math.isclose(num, dg[c], rel_tol=1e-6, abs_tol=1e-8)


def test_layernorm_memory_efficient_equals_plain_when_gamma_is_large():
    x, gamma, beta, dy = _ln_inputs(4, 16, 3)
    eps = 1e-5
    y, mean, _, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    plain = oracle.layernorm_bwd(dy, x, gamma, mean, rstd, eps, clamp_gamma=True)
    # hand the exact y to the memory-efficient variant through float64 -> it takes float32: use y rounded, loose tol
    me = oracle.layernorm_bwd_memeff(dy, y.astype(np.float32), gamma, beta, rstd, eps)
    for a, b in zip(plain, me):
        assert np.allclose(a, b, rtol=1e-5, atol=1e-5)
    # clamp_by_magnitude: |gamma| < eps is pushed to +-eps, zero counts as positive
    g2 = gamma.copy(); g2[:3] = [1e-9, -1e-9, 0.0]
    dxa, _, _ = oracle.layernorm_bwd(dy, x, g2, mean, rstd, eps, clamp_gamma=True)
    dxb, _, _ = oracle.layernorm_bwd(dy, x, g2, mean, rstd, eps, clamp_gamma=False)
    assert not np.allclose(dxa[:, :3], dxb[:, :3]) and np.allclose(dxa[:, 3:], dxb[:, 3:], **F64)
    s1 = (dy.astype(np.float64) * g2).sum(1); xh = (x - mean[:, None]) * rstd[:, None]
    s2 = (dy.astype(np.float64) * g2 * xh).sum(1)
    want0 = rstd / 16 * (16 * dy[:, 0].astype(np.float64) * eps - s1 - xh[:, 0] * s2)
    assert np.allclose(dxa[:, 0], want0, **F64)


# ---------------------------------------------------------------------------
# RMSNorm / dropout-add-LN (flash-attention layer_norm arithmetic)
# ---------------------------------------------------------------------------
def test_rmsnorm_closed_form_and_torch():
    x, gamma, _, dz = _ln_inputs(6, 32, 4)
    eps = 1e-6
    z, _, mu, rs = oracle.dropout_add_ln_fwd(x, None, gamma, None, eps, True)
    xd = x.astype(np.float64)
    assert np.allclose(rs, 1 / np.sqrt((xd ** 2).mean(1) + eps), **F64)    # var + mu^2 = mean(x^2)
    assert np.allclose(mu, xd.mean(1), **F64)
    assert np.allclose(z, xd * rs[:, None] * gamma, **F64)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tg = torch.tensor(gamma, dtype=torch.float64, requires_grad=True)
    tz = tx * torch.rsqrt((tx * tx).mean(1, keepdim=True) + eps) * tg
    tz.backward(torch.tensor(dz, dtype=torch.float64))
    dx, dg, db = oracle.dropout_add_ln_bwd(dz, None, x, mu, rs, gamma, True)
    assert np.allclose(dx, tx.grad.numpy(), **F64) and np.allclose(dg, tg.grad.numpy(), **F64)
    assert np.allclose(db, dz.astype(np.float64).sum(0), **F64)
    # sum_cols dx*x = eps * rs^3 * sum_cols (gamma*dz)*x : exactly zero only for eps = 0
    lhs = (dx * xd).sum(1)
    rhs = eps * rs ** 3 * (gamma * dz.astype(np.float64) * xd).sum(1)
    assert np.allclose(lhs, rhs, rtol=1e-6, atol=1e-12)


def test_dropout_add_ln_layernorm_mode_and_residual():
    x0, gamma, beta, dz = _ln_inputs(5, 16, 5)
    res = np.random.default_rng(6).standard_normal((5, 16)).astype(np.float32)
    eps = 1e-5
    z, xo, mu, rs = oracle.dropout_add_ln_fwd(x0, res, gamma, beta, eps, False)
    xs = x0.astype(np.float64) + res
    assert np.allclose(xo, xs, **F64)
    y2, mean2, _, rstd2 = oracle.layernorm_fwd(xs.astype(np.float32), gamma, beta, eps)
    assert np.allclose(mu, xs.mean(1), **F64)
    tx = torch.tensor(xs, dtype=torch.float64, requires_grad=True)
    tz = torch.nn.functional.layer_norm(tx, (16,), torch.tensor(gamma, dtype=torch.float64),
                                        torch.tensor(beta, dtype=torch.float64), eps)
    assert np.allclose(z, tz.detach().numpy(), **F64)
    tz.backward(torch.tensor(dz, dtype=torch.float64))
    dxin = np.random.default_rng(7).standard_normal((5, 16)).astype(np.float32)
    # backward consumes x as stored (float32): rebuild expectations from that x
    xst = xs.astype(np.float32)
    dx, dg, db = oracle.dropout_add_ln_bwd(dz, dxin, xst, xst.astype(np.float64).mean(1),
                                           1 / np.sqrt(xst.astype(np.float64).var(1) + eps), gamma, False)
    assert np.allclose(dx - dxin, tx.grad.numpy(), rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------
# Softmax
# ---------------------------------------------------------------------------
def test_softmax_properties_and_torch():
    g = np.random.default_rng(8)
    x = (g.standard_normal((3, 5, 7)) * 3).astype(np.float32)
    for dim in (0, 1, 2, -1):
        y = oracle.softmax_fwd(x, dim)
        assert np.allclose(y.sum(dim), 1.0, **F64)
        assert np.allclose(y, torch.softmax(torch.tensor(x, dtype=torch.float64), dim).numpy(), **F64)
        dy = g.standard_normal(x.shape).astype(np.float32)
        dx = oracle.softmax_bwd(y.astype(np.float32), dy, dim)
        ty = torch.tensor(y.astype(np.float32), dtype=torch.float64)
        want = ty * (torch.tensor(dy, dtype=torch.float64) - (ty * torch.tensor(dy, dtype=torch.float64)).sum(dim, keepdim=True))
        assert np.allclose(dx, want.numpy(), **F64)
        assert np.allclose(dx.sum(dim), 0, atol=1e-6)
    # shift invariance with exactly representable shifts, one-hot limit, all-equal rows
    xs = np.round(x * 8) / 8
    assert np.allclose(oracle.softmax_fwd(xs + 64.0), oracle.softmax_fwd(xs), **F64)
    one = np.full((1, 9), -200.0, np.float32); one[0, 4] = 50.0
    y = oracle.softmax_fwd(one)
    assert y[0, 4] == 1.0 and y.sum() == 1.0
    assert np.allclose(oracle.softmax_fwd(np.full((2, 10), 3.0, np.float32)), 0.1, **F64)
    # brute force
    row = [0.5, -1.25, 2.0, 0.0]
    den = sum(math.exp(v) for v in row)
    assert np.allclose(oracle.softmax_fwd(np.array([row], np.float32))[0], [math.exp(v) / den for v in row], **F64)


# ---------------------------------------------------------------------------
# Softmax cross-entropy
# ---------------------------------------------------------------------------
def test_sce_sparse_closed_form_torch_and_ignore():
    g = np.random.default_rng(9)
    rows, cols, ign = 12, 9, -100
    x = (g.standard_normal((rows, cols)) * 2).astype(np.float32)
    lab = g.integers(0, cols, rows).astype(np.int64)
    lab[[2, 7]] = ign
    loss = oracle.sce_sparse_fwd(x, lab, ign)
    xd = x.astype(np.float64)
    for r in range(rows):                                     # brute force
        want = 0.0 if lab[r] == ign else math.log(sum(math.exp(v) for v in xd[r])) - xd[r, lab[r]]
        assert math.isclose(loss[r], want, rel_tol=1e-12, abs_tol=1e-12)
    assert loss[2] == 0.0 and loss[7] == 0.0
    tl = torch.nn.functional.cross_entropy(torch.tensor(xd), torch.tensor(lab), ignore_index=ign, reduction="none")
    assert np.allclose(loss, tl.numpy(), **F64)
    # Hetu's mean divides by ALL rows; torch's by the valid ones: rescale by n_valid / rows
    tmean = torch.nn.functional.cross_entropy(torch.tensor(xd), torch.tensor(lab), ignore_index=ign).item()
    assert math.isclose(loss.sum() / rows, tmean * (rows - 2) / rows, rel_tol=1e-12)
    gl = (g.random(rows) + 0.5).astype(np.float32)
    dx = oracle.sce_sparse_bwd(x, lab, gl, ign)
    tx = torch.tensor(xd, requires_grad=True)
    (torch.nn.functional.cross_entropy(tx, torch.tensor(lab), ignore_index=ign, reduction="none")
     * torch.tensor(gl, dtype=torch.float64)).sum().backward()
    assert np.allclose(dx, tx.grad.numpy(), **F64)
    assert np.all(dx[[2, 7]] == 0.0)
    valid = lab != ign
    assert np.allclose(dx[valid].sum(1), 0, atol=1e-12)


def test_sce_dense_matches_sparse_on_one_hot_and_torch():
    g = np.random.default_rng(10)
    rows, cols = 6, 11
    x = (g.standard_normal((rows, cols)) * 2).astype(np.float32)
    lab = g.integers(0, cols, rows).astype(np.int64)
    onehot = np.eye(cols, dtype=np.float32)[lab]
    assert np.allclose(oracle.sce_dense_fwd(x, onehot), oracle.sce_sparse_fwd(x, lab, -1), **F64)
    gl = (g.random(rows) + 0.5).astype(np.float32)
    assert np.allclose(oracle.sce_dense_bwd(x, onehot, gl), oracle.sce_sparse_bwd(x, lab, gl, -1), **F64)
    soft = g.random((rows, cols)).astype(np.float32)
    soft /= soft.sum(1, keepdims=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tl = -(torch.tensor(soft, dtype=torch.float64) * torch.log_softmax(tx, 1)).sum(1)
    assert np.allclose(oracle.sce_dense_fwd(x, soft), tl.detach().numpy(), **F64)
    (tl * torch.tensor(gl, dtype=torch.float64)).sum().backward()
    # dx = (softmax - label) * g holds when the labels of a row sum to one (float32 rounding of `soft` aside)
    assert np.allclose(oracle.sce_dense_bwd(x, soft, gl), tx.grad.numpy(), rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------------------
# Reduce
# ---------------------------------------------------------------------------
def test_reduce_every_axis_subset_and_axis_handling():
    import itertools
    x = np.random.default_rng(11).integers(-3, 4, size=(3, 4, 5, 6)).astype(np.float64)
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            want = x.sum(axis=axes)
            got = oracle.reduce(x, list(axes), "sum")
            assert np.array_equal(got.reshape(-1), np.asarray(want).reshape(-1))
            assert np.allclose(oracle.reduce(x, list(axes), "mean").reshape(-1), np.asarray(x.mean(axis=axes)).reshape(-1), **F64)
    assert np.array_equal(oracle.reduce(x, [2, 0, 2], "sum"), x.sum(axis=(0, 2)))     # unsorted + repeated axes
    # strided view: transpose described by strides only
    base = np.arange(24, dtype=np.float64)
    got = oracle.strided_reduce(base, [4, 6], [1, 4], [0], "sum")                        # view = base.reshape(6,4).T
    assert np.array_equal(got, base.reshape(6, 4).T.sum(0))
    with pytest.raises(ValueError):
        oracle.strided_reduce(base, [4, 6], [6, 1], [2], "sum")


def test_reduce_mean_rounding_modes():
    x = np.random.default_rng(12).integers(-8, 9, size=(4, 3000)).astype(np.float64)
    exact = oracle.reduce(x, [1], "mean", mean_mode=0)
    ref = oracle.reduce(x, [1], "mean", mean_mode=1)
    want = (x.sum(1).astype(np.float32) * (np.float32(1.0) / np.float32(3000))).astype(np.float64)
    assert np.array_equal(ref, want)                       # fp32 sum * fp32(1/n), as the reference orders it
    assert np.allclose(ref, exact, rtol=2e-7)


def test_reduce_max_min_prod_against_numpy_and_nan_rule():
    """Selections are exact; a NaN anywhere in the reduced set wins (numpy's max / min have the same rule);
    identities are -inf, +inf and 1 (an empty reduced extent); products against numpy float64."""
    import itertools
    g = np.random.default_rng(14)
    x = g.standard_normal((3, 4, 5, 6))
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            for op, f in (("max", np.max), ("min", np.min)):
                assert np.array_equal(oracle.reduce(x, list(axes), op).reshape(-1), np.asarray(f(x, axis=axes)).reshape(-1))
            assert np.allclose(oracle.reduce(x, list(axes), "prod").reshape(-1), np.asarray(np.prod(x, axis=axes)).reshape(-1), **F64)
    y = x.copy()
    y[1, 2, 3, 4] = np.nan
    for op, f in (("max", np.max), ("min", np.min)):
        got, want = oracle.reduce(y, [1, 3], op), f(y, axis=(1, 3))
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(got).sum() == 1
        assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    empty = np.zeros((4, 0))
    assert np.all(oracle.reduce(empty, [1], "max") == -np.inf)
    assert np.all(oracle.reduce(empty, [1], "min") == np.inf)
    assert np.all(oracle.reduce(empty, [1], "prod") == 1.0)
    assert np.all(oracle.reduce(empty, [1], "sum") == 0.0)
    # all-equal and single-element rows
    assert np.array_equal(oracle.reduce(np.full((3, 7), -2.5), [1], "max"), np.full(3, -2.5))
    assert np.array_equal(oracle.reduce(x[:, :1], [1], "min").reshape(-1), x[:, 0].reshape(-1))


def test_nll_loss_is_the_cross_entropy_of_log_softmax():
    """NLL(log_softmax(x)) is the sparse cross-entropy; its gradient routed through the reference's
    scaling (-grad * cols at the label) is a one-hot pattern; out-of-range labels give 0 / an all-zero row."""
    import torch
    g = np.random.default_rng(15)
    x = g.standard_normal((9, 40))
    lab = g.integers(0, 40, size=9)
    logp = torch.log_softmax(torch.from_numpy(x), dim=1).numpy()
    assert np.allclose(oracle.nll_loss_fwd(logp, lab), oracle.sce_sparse_fwd(x.astype(np.float32).astype(np.float64).astype(np.float32), lab, -100), rtol=1e-5, atol=1e-6)
    assert np.allclose(oracle.nll_loss_fwd(logp, lab), torch.nn.functional.nll_loss(torch.from_numpy(logp), torch.from_numpy(lab), reduction="none").numpy(), **F64)
    lab2 = lab.copy(); lab2[0] = -1; lab2[1] = 40
    assert oracle.nll_loss_fwd(logp, lab2)[0] == 0.0 and oracle.nll_loss_fwd(logp, lab2)[1] == 0.0
    gl = g.standard_normal(9)
    out = oracle.nll_loss_bwd(lab2, gl, 40)
    assert np.count_nonzero(out) == 7 and not out[0].any() and not out[1].any()
    for r in range(2, 9):
        assert out[r, lab2[r]] == -gl[r] * 40


# ---------------------------------------------------------------------------
# fp32 CPU ports (the timed baseline) agree with the float64 oracle
# ---------------------------------------------------------------------------
def test_refcpu_ports_match_oracle():
    import ctypes
    lib = oracle.lib()
    g = np.random.default_rng(13)
    rows, cols = 33, 512
    x = g.standard_normal((rows, cols)).astype(np.float32)
    gamma = (g.random(cols) + 0.5).astype(np.float32); beta = (g.standard_normal(cols) * .1).astype(np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    P = lambda a: a.ctypes.data_as(fp)
    R, C = ctypes.c_int64(rows), ctypes.c_int64(cols)
    y = np.empty_like(x); mean = np.empty(rows, np.float32); var = np.empty(rows, np.float32)
    lib.refcpu_layernorm_fwd_f32(P(x), P(gamma), P(beta), R, C, ctypes.c_float(1e-5), P(y), P(mean), P(var))
    ey, em, ev, _ = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
    assert np.allclose(y, ey, rtol=1e-4, atol=1e-5) and np.allclose(var, ev, rtol=1e-4)
    z = np.empty_like(x); rs = np.empty(rows, np.float32)
    lib.refcpu_rmsnorm_fwd_f32(P(x), P(gamma), R, C, ctypes.c_float(1e-6), P(z), P(rs))
    ez, _, _, ers = oracle.dropout_add_ln_fwd(x, None, gamma, None, 1e-6, True)
    assert np.allclose(z, ez, rtol=1e-4, atol=1e-5) and np.allclose(rs, ers, rtol=1e-5)
    dz = g.standard_normal((rows, cols)).astype(np.float32)
    dx = np.empty_like(x); dg = np.empty(cols, np.float32)
    lib.refcpu_rmsnorm_bwd_f32(P(dz), P(x), P(gamma), P(rs), R, C, P(dx), P(dg))
    edx, edg, _ = oracle.dropout_add_ln_bwd(dz, None, x, None, rs, gamma, True)
    assert np.allclose(dx, edx, rtol=1e-3, atol=1e-4) and np.allclose(dg, edg, rtol=1e-3, atol=1e-3)
    sm = np.empty_like(x)
    lib.refcpu_softmax_fwd_f32(P(x), R, C, P(sm))
    assert np.allclose(sm, oracle.softmax_fwd(x), rtol=1e-5, atol=1e-8)
    lab = g.integers(0, cols, rows).astype(np.int64); lab[3] = -100
    loss = np.empty(rows, np.float32)
    lib.refcpu_sce_sparse_fwd_f32(P(x), lab.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), R, C, ctypes.c_int64(-100), P(loss))
    assert np.allclose(loss, oracle.sce_sparse_fwd(x, lab, -100), rtol=1e-5, atol=1e-5)
    out1 = np.empty(rows, np.float32); out0 = np.empty(cols, np.float32)
    lib.refcpu_reduce_sum_axis1_f32(P(x), R, C, P(out1)); lib.refcpu_reduce_sum_axis0_f32(P(x), R, C, P(out0))
    assert np.allclose(out1, x.astype(np.float64).sum(1), atol=1e-3) and np.allclose(out0, x.astype(np.float64).sum(0), atol=1e-3)
    lib.refcpu_reduce_mean_axis1_f32(P(x), R, C, P(out1)); lib.refcpu_reduce_mean_axis0_f32(P(x), R, C, P(out0))
    assert np.allclose(out1, x.astype(np.float64).mean(1), atol=1e-5) and np.allclose(out0, x.astype(np.float64).mean(0), atol=1e-5)
    # LayerNorm gradient in the reference's pass structure (statistics: mean and variance) against the float64 oracle
    dy = g.standard_normal((rows, cols)).astype(np.float32)
    _, em, ev, erstd = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
    mean32, var32 = em.astype(np.float32), ev.astype(np.float32)
    dxl = np.empty_like(x); dgl = np.empty(cols, np.float32); dbl = np.empty(cols, np.float32)
    lib.refcpu_layernorm_bwd_f32(P(dy), P(x), P(gamma), P(mean32), P(var32), R, C, ctypes.c_float(1e-5), P(dxl), P(dgl), P(dbl))
    edx, edg, edb = oracle.layernorm_bwd(dy, x, gamma, em, erstd)
    assert np.allclose(dxl, edx, rtol=1e-3, atol=1e-4) and np.allclose(dgl, edg, rtol=1e-3, atol=1e-3)
    assert np.allclose(dbl, edb, rtol=1e-4, atol=1e-4)
    # sparse cross-entropy gradient: ignored row all zeros, the rest against the float64 oracle
    gl = g.standard_normal(rows).astype(np.float32)
    dxc = np.empty_like(x)
    lib.refcpu_sce_sparse_bwd_f32(P(x), lab.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), P(gl), R, C, ctypes.c_int64(-100), P(dxc))
    assert not dxc[3].any()
    assert np.allclose(dxc, oracle.sce_sparse_bwd(x, lab, gl, -100), rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("p", [1, 2, 3, 4])
@pytest.mark.parametrize("dim", [0, 1, 2])
def test_p_norm_against_torch_autograd(p, dim):
    """oracle.norm_p_fwd / norm_p_bwd against torch.linalg.vector_norm and its float64 autograd (an independent
    implementation); the zero slice by the definition (gradient 0, sign(0) = 0)."""
    import torch
    g = np.random.default_rng(10 * p + dim)
    x = g.standard_normal((4, 5, 6))
    x[1, 2, 3] = 0.0                      # an exact zero inside a non-zero slice
    grad = g.standard_normal(tuple(s for i, s in enumerate(x.shape) if i != dim))
    n = oracle.norm_p_fwd(x, dim, p)
    tx = torch.tensor(x, requires_grad=True)
    tn = torch.linalg.vector_norm(tx, ord=p, dim=dim)
    np.testing.assert_allclose(n, tn.detach().numpy(), rtol=1e-13)
    (tn * torch.tensor(grad)).sum().backward()
    np.testing.assert_allclose(oracle.norm_p_bwd(x, n, grad, dim, p), tx.grad.numpy(), rtol=1e-11, atol=1e-13)
    z = np.zeros((2, 3, 4))
    nz = oracle.norm_p_fwd(z, dim, p)
    assert (nz == 0).all()
    gz = np.ones(nz.shape)
    assert (oracle.norm_p_bwd(z, nz, gz, dim, p) == 0).all()


def test_batch_norm_against_torch():
    """oracle.batch_norm_fwd / _bwd against torch.nn.functional.batch_norm in training mode (float64; its
    running-variance update also takes the unbiased estimate) and torch autograd."""
    import torch
    g = np.random.default_rng(5)
    x = g.standard_normal((6, 5, 4, 3)) * 2 + 1
    scale = g.uniform(0.5, 1.5, 5); bias = g.standard_normal(5)
    rm = g.standard_normal(5); rv = g.uniform(0.5, 2.0, 5)
    dy = g.standard_normal(x.shape)
    y, nrm, nrv, smean, sinv = oracle.batch_norm_fwd(x, scale, bias, rm, rv, 0.1, 1e-5)
    tx = torch.tensor(x, requires_grad=True); ts = torch.tensor(scale, requires_grad=True)
    tb = torch.tensor(bias, requires_grad=True)
    trm, trv = torch.tensor(rm), torch.tensor(rv)
    ty = torch.nn.functional.batch_norm(tx, trm, trv, ts, tb, training=True, momentum=0.1, eps=1e-5)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(nrm, trm.numpy(), rtol=1e-13)
    np.testing.assert_allclose(nrv, trv.numpy(), rtol=1e-13)
    np.testing.assert_allclose(smean, x.mean(axis=(0, 2, 3)), rtol=1e-13)
    np.testing.assert_allclose(sinv, 1 / np.sqrt(x.var(axis=(0, 2, 3)) + 1e-5), rtol=1e-13)
    (ty * torch.tensor(dy)).sum().backward()
    dx, dscale, dbias = oracle.batch_norm_bwd(dy, x, scale, smean, sinv)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dscale, ts.grad.numpy(), rtol=1e-11)
    np.testing.assert_allclose(dbias, tb.grad.numpy(), rtol=1e-11)


@pytest.mark.parametrize("case", [
    ((4, 5), (3, 4, 5), ()), ((1, 5), (3, 4, 5), ()), ((1,), (2, 3), ()), ((4, 1), (3, 4, 5), ()),
    ((3, 5), (3, 4, 5), (1,)), ((4,), (3, 4, 5), (0, 2)), ((3,), (3, 4, 5), (1, 2)), ((5,), (3, 4, 5), (0, 1)),
    ((3, 1, 5), (3, 4, 5), (1,)),     # keepdims: no dimension to add, the axis list is not consulted
], ids=str)
def test_broadcast_shape_is_numpy_broadcasting(case):
    """oracle.broadcast_shape's index arithmetic against numpy's own broadcasting, with the dropped dimensions put
    back by expand_dims (an independent statement of the same layout), and against torch autograd of sum / mean,
    whose gradient is this broadcast (times 1/n for the mean)."""
    import torch
    in_shape, out_shape, add_axes = case
    g = np.random.default_rng(len(in_shape) * 7 + len(add_axes))
    x = g.standard_normal(in_shape)
    diff = len(out_shape) - len(in_shape)
    want = np.broadcast_to(np.expand_dims(x, tuple(add_axes[:diff])) if add_axes else x, out_shape)
    np.testing.assert_array_equal(oracle.broadcast_shape(x, out_shape, add_axes), want)
    np.testing.assert_allclose(oracle.broadcast_shape(x, out_shape, add_axes, 0.25), want * 0.25, rtol=0)
    if add_axes and diff == len(add_axes):
        t = torch.zeros(out_shape, dtype=torch.float64, requires_grad=True)
        (t.mean(dim=tuple(add_axes)) * torch.tensor(x)).sum().backward()
        n = np.prod([out_shape[a] for a in add_axes])
        np.testing.assert_allclose(oracle.broadcast_shape(x, out_shape, add_axes, 1.0 / n), t.grad.numpy(),
                                   rtol=1e-15)
