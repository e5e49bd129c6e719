"""Pins oracle/dropout_add_ln.py (the numpy restatement of the full dropout-add-LayerNorm interface):
Philox4x32-10 against the Random123 known-answer vectors, the uniform map against curand_uniform's closed
form, every output and gradient against torch (float64 autograd of the composed function, an independent
implementation), and the feature-free case against the plain norm oracle."""
import numpy as np
import pytest
import torch

import oracle
from oracle import dropout_add_ln as dal


def test_philox_known_answers():
    # kat_vectors of the Random123 distribution, philox4x32 with 10 rounds
    cases = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for ctr, key, want in cases:
        got = dal.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
        assert [int(v) for v in got] == want
    # vectorised call == one call per counter
    ctr = np.array([[i, 3, 5, 7] for i in range(9)], dtype=np.uint32)
    key = np.array([11, 13], dtype=np.uint32)
    batch = dal.philox4x32_10(ctr, key)
    for i in range(9):
        assert (batch[i] == dal.philox4x32_10(ctr[i], key)).all()


def test_uniform_map_and_mask():
    u = dal.uniform_from_bits([0, 1 << 31, 0xffffffff, 1])
    assert u[0] == np.float32(2.0 ** -33) and u[1] == np.float32(0.5) and u[2] == np.float32(1.0)
    assert u[3] == np.float32(2.0 ** -32 + 2.0 ** -33)
    assert (dal.uniform_from_bits(np.arange(0, 1 << 32, 65521, dtype=np.uint64)) > 0).all()
    # a draw of exactly 1.0 is dropped for every p > 0; everything is kept at p = 0
    assert dal.dropout_keep(5, 0, 4096, 1.0).all()
    n = 1 << 20
    for p in (0.1, 0.5):
        keep = dal.dropout_keep(42, 3, n, 1.0 - p)
        sigma = np.sqrt(p * (1 - p) / n)
        assert abs(keep.mean() - (1 - p)) < 5 * sigma
    # streams differ by seed, offset and input number; a prefix does not depend on the length
    a = dal.dropout_keep(42, 3, 4096, 0.5)
    assert (a[:1001] == dal.dropout_keep(42, 3, 1001, 0.5)).all()
    for other in (dal.dropout_keep(43, 3, 4096, 0.5), dal.dropout_keep(42, 4, 4096, 0.5),
                  dal.dropout_keep(42, 3, 4096, 0.5, which=1)):
        assert 0.4 < (a != other).mean() < 0.6


def _torch_norm(x, gamma, beta, eps, is_rms):
    if is_rms:
        y = x * torch.rsqrt((x * x).mean(dim=1, keepdim=True) + eps)
    else:
        mu = x.mean(dim=1, keepdim=True)
        y = (x - mu) * torch.rsqrt(((x - mu) ** 2).mean(dim=1, keepdim=True) + eps)
    z = y * gamma
    return z + beta if beta is not None else z


@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("features", ["plain", "dropout", "rowscale", "colscale", "dropout+colscale+residual",
                                      "all"])
def test_fwd_bwd_against_torch_autograd(is_rms, features):
    rng = np.random.default_rng(sum(map(ord, features)) + int(is_rms))
    rows, cols, eps = 7, 24, 1e-5
    p = 0.25 if "dropout" in features or features == "all" else 0.0
    x0 = rng.standard_normal((rows, cols)); gamma = rng.uniform(0.5, 1.5, cols); beta = rng.standard_normal(cols)
    residual = rng.standard_normal((rows, cols)) if ("residual" in features or features == "all") else None
    rowscale = rng.uniform(0.5, 2.0, rows) if features in ("rowscale", "all") else None
    colscale = rng.uniform(0.5, 2.0, cols) if ("colscale" in features or features == "all") else None
    dmask = dal.dropout_keep(9, 1, rows * cols, 1 - p).reshape(rows, cols) if p > 0 else None
    dz = rng.standard_normal((rows, cols)); dx_in = rng.standard_normal((rows, cols))

    z, x, mu, rs = dal.fwd(x0, residual, gamma, None if is_rms else beta, rowscale, colscale, dmask=dmask,
                           dropout_p=p, eps=eps, is_rms=is_rms)
    dx0, dres, dg, db, dcol = dal.bwd(dz, dx_in, x, x0, dmask, mu, rs, gamma, rowscale, colscale,
                                      dropout_p=p, is_rms=is_rms)

    T = lambda a: None if a is None else torch.tensor(a, dtype=torch.float64)
    tx0 = T(x0).requires_grad_(True); tg = T(gamma).requires_grad_(True); tb = T(beta).requires_grad_(True)
    tres = T(residual).requires_grad_(True) if residual is not None else None
    tcs = T(colscale).requires_grad_(True) if colscale is not None else None
    v = tx0
    if rowscale is not None:
        v = v * T(rowscale)[:, None]
    if p > 0:
        v = v * T(dmask.astype(np.float64)) / (1 - p)
    if tcs is not None:
        v = v * tcs
    tx = v + tres if tres is not None else v
    tx.retain_grad()
    tz = _torch_norm(tx, tg, None if is_rms else tb, eps, is_rms)
    # the upstream gradient of the pre-norm sum enters as an extra linear term
    (tz * T(dz)).sum().add((tx * T(dx_in)).sum()).backward()

    np.testing.assert_allclose(z, tz.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(x, tx.detach().numpy(), rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(mu, tx.detach().numpy().mean(axis=1), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dx0, tx0.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dres, tx.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-10, atol=1e-11)
    if not is_rms:
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-10, atol=1e-11)
    if colscale is not None:
        np.testing.assert_allclose(dcol, tcs.grad.numpy(), rtol=1e-10, atol=1e-11)
    if residual is not None:
        np.testing.assert_allclose(dres, tres.grad.numpy(), rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("p", [0.0, 0.3])
def test_subset_against_torch_autograd(is_rms, p):
    """Row subsets: row r of the normalised sum reads x0 row x0_subset[r]-1 (0: nothing) and writes z row
    z_subset[r]-1 (0: not written); composed in torch with gathers."""
    rng = np.random.default_rng(3 + int(is_rms))
    rows, cols, eps, x0_rows, z_rows, rsc = 6, 16, 1e-5, 4, 3, 0.7
    x0_subset = np.array([1, 0, 3, 4, 0, 2], dtype=np.int32)
    z_subset = np.array([0, 1, 2, 0, 3, 0], dtype=np.int32)
    x0 = rng.standard_normal((x0_rows, cols)); residual = rng.standard_normal((rows, cols))
    gamma = rng.uniform(0.5, 1.5, cols); beta = rng.standard_normal(cols); colscale = rng.uniform(0.5, 2.0, cols)
    dmask = dal.dropout_keep(1, 0, x0_rows * cols, 1 - p).reshape(x0_rows, cols) if p > 0 else None
    dz = rng.standard_normal((z_rows, cols)); dx_in = rng.standard_normal((rows, cols))

    z, x, mu, rs = dal.fwd(x0, residual, gamma, beta, None, colscale, x0_subset, z_subset, dmask, p, eps, rsc,
                           z_rows, is_rms)
    dx0, dres, dg, db, dcol = dal.bwd(dz, dx_in, x, x0, dmask, mu, rs, gamma, None, colscale, x0_subset,
                                      z_subset, p, rsc, x0_rows, is_rms)

    T = lambda a: torch.tensor(a, dtype=torch.float64)
    tx0 = T(x0).requires_grad_(True); tg = T(gamma).requires_grad_(True); tb = T(beta).requires_grad_(True)
    tcs = T(colscale).requires_grad_(True); tres = T(residual).requires_grad_(True)
    v = tx0 * rsc
    if p > 0:
        v = v * T(dmask.astype(np.float64)) / (1 - p)
    v = v * tcs
    picked = torch.zeros(rows, cols, dtype=torch.float64)
    has = torch.tensor(x0_subset > 0)
    picked = torch.where(has[:, None], v[torch.tensor(np.maximum(x0_subset - 1, 0), dtype=torch.long)], picked)
    tx = picked + tres
    tx.retain_grad()
    tzfull = _torch_norm(tx, tg, tb, eps, is_rms)
    loss = (tx * T(dx_in)).sum()
    for r in range(rows):
        if z_subset[r] > 0:
            loss = loss + (tzfull[r] * T(dz[z_subset[r] - 1])).sum()
            np.testing.assert_allclose(z[z_subset[r] - 1], tzfull[r].detach().numpy(), rtol=1e-12, atol=1e-12)
    loss.backward()
    np.testing.assert_allclose(x, tx.detach().numpy(), rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(dx0, tx0.grad.numpy(), rtol=1e-10, atol=1e-11)   # every x0 row is referenced
    np.testing.assert_allclose(dres, tres.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dcol, tcs.grad.numpy(), rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("has_x1,tied,p", [(True, False, 0.2), (True, True, 0.0), (False, False, 0.2),
                                           (False, True, 0.0)])
def test_parallel_residual_against_torch_autograd(is_rms, has_x1, tied, p):
    rng = np.random.default_rng(11 + int(is_rms) + 2 * int(has_x1) + 4 * int(tied))
    rows, cols, eps = 5, 16, 1e-5
    x0 = rng.standard_normal((rows, cols)); x1 = rng.standard_normal((rows, cols)) if has_x1 else None
    residual = rng.standard_normal((rows, cols))
    g0 = rng.uniform(0.5, 1.5, cols); b0 = rng.standard_normal(cols)
    g1 = None if tied else rng.uniform(0.5, 1.5, cols); b1 = None if tied else rng.standard_normal(cols)
    m0 = dal.dropout_keep(2, 5, rows * cols, 1 - p).reshape(rows, cols) if p > 0 else None
    m1 = dal.dropout_keep(2, 5, rows * cols, 1 - p, which=1).reshape(rows, cols) if p > 0 and has_x1 else None
    dz0 = rng.standard_normal((rows, cols)); dz1 = None if tied else rng.standard_normal((rows, cols))
    dx_in = rng.standard_normal((rows, cols))

    z0, z1, x, mu, rs = dal.parallel_fwd(x0, x1, residual, g0, b0, g1, b1, m0, m1, p, eps, is_rms)
    dx0, dx1, dres, dg0, db0, dg1, db1 = dal.parallel_bwd(dz0, dz1, dx_in, x, m0, m1, mu, rs, g0, g1, p, has_x1,
                                                          is_rms)

    T = lambda a: torch.tensor(a, dtype=torch.float64)
    tx0 = T(x0).requires_grad_(True); tres = T(residual).requires_grad_(True)
    tg0 = T(g0).requires_grad_(True); tb0 = T(b0).requires_grad_(True)
    v = tx0 * T(m0.astype(np.float64)) / (1 - p) if p > 0 else tx0
    if has_x1:
        tx1 = T(x1).requires_grad_(True)
        v = v + (tx1 * T(m1.astype(np.float64)) / (1 - p) if p > 0 else tx1)
    tx = v + tres
    tz0 = _torch_norm(tx, tg0, tb0, eps, is_rms)
    loss = (tz0 * T(dz0)).sum() + (tx * T(dx_in)).sum()
    if not tied:
        tg1 = T(g1).requires_grad_(True); tb1 = T(b1).requires_grad_(True)
        tz1 = _torch_norm(tx, tg1, tb1, eps, is_rms)
        loss = loss + (tz1 * T(dz1)).sum()
        np.testing.assert_allclose(z1, tz1.detach().numpy(), rtol=1e-12, atol=1e-12)
    else:
        assert z1 is None and dg1 is None and db1 is None
    loss.backward()
    np.testing.assert_allclose(z0, tz0.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dx0, tx0.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dres, tres.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(dg0, tg0.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(db0, tb0.grad.numpy(), rtol=1e-10, atol=1e-11)
    if has_x1:
        np.testing.assert_allclose(dx1, tx1.grad.numpy(), rtol=1e-10, atol=1e-11)
    else:
        assert dx1 is None
    if not tied:
        np.testing.assert_allclose(dg1, tg1.grad.numpy(), rtol=1e-10, atol=1e-11)
        np.testing.assert_allclose(db1, tb1.grad.numpy(), rtol=1e-10, atol=1e-11)


def test_feature_free_case_is_the_plain_norm_oracle():
    rng = np.random.default_rng(0)
    x0 = rng.standard_normal((9, 32)).astype(np.float32); res = rng.standard_normal((9, 32)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 32).astype(np.float32); b = rng.standard_normal(32).astype(np.float32)
    for is_rms in (False, True):
        z, x, mu, rs = dal.fwd(x0, res, g, None if is_rms else b, eps=1e-6, is_rms=is_rms)
        ez, ex, emu, ers = oracle.dropout_add_ln_fwd(x0, res, g, None if is_rms else b, 1e-6, is_rms)
        np.testing.assert_allclose(z, ez, rtol=1e-11, atol=1e-12)
        np.testing.assert_allclose(x, ex, rtol=0, atol=0)
        np.testing.assert_allclose(mu, emu, rtol=1e-12, atol=1e-14)
        np.testing.assert_allclose(rs, ers, rtol=1e-12)
