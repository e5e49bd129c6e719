"""GPU parity of the fused softmax cross-entropy kernels (hk_sce_*)."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

IGN = -100


def _labels(rows, cols, seed, frac=0.05):
    g = helpers.rng(seed)
    lab = g.integers(0, cols, size=rows, dtype=np.int64)
    lab[g.random(rows) < frac] = IGN
    return lab


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape", [(9, 64), (33, 1000), (17, 32000), (5, 7), (64, 4096), (3, 50257), (2, 131072 + 8)])
def test_sce_sparse(hk, cuda, dtype, shape):
    import torch
    rows, cols = shape
    x = helpers.draw(501, shape, "normal", 0.0, 2.0, dtype)
    lab = _labels(rows, cols, 502, 0.2)
    lab[0] = cols - 1
    eloss = oracle.sce_sparse_fwd(x, lab, IGN)
    tx = helpers.to_torch(x, dtype, cuda)
    tl = torch.from_numpy(lab).to(cuda)
    tloss = torch.full((rows,), 7.0, dtype=tx.dtype, device=cuda)
    hk.sce_sparse_fwd(tx, tl, tloss, IGN)
    torch.cuda.synchronize()
    helpers.assert_close(tloss, eloss, dtype, "loss")
    ign = lab == IGN
    # ignored rows: exactly +0.0 bits
    assert torch.all(tloss.view(torch.int16 if dtype != "fp32" else torch.int32)[torch.from_numpy(ign).to(cuda)] == 0)

    g = helpers.draw(503, (rows,), "uniform", 0.5, 1.5, dtype) / np.float32(rows)
    g = oracle.round_to(g, dtype)
    edx = oracle.sce_sparse_bwd(x, lab, g, IGN)
    tg = helpers.to_torch(g, dtype, cuda)
    tdx = torch.full_like(tx, 3.0)
    hk.sce_sparse_bwd(tx, tl, tg, tdx, IGN)
    torch.cuda.synchronize()
    helpers.assert_close(tdx, edx, dtype, "dlogits")
    if ign.any():
        assert torch.count_nonzero(tdx[torch.from_numpy(ign).to(cuda)]) == 0   # zero rows, bit exact
    # valid rows sum to ~0 (softmax sums to one)
    rs = tdx.float().sum(1).abs().cpu().numpy()
    assert np.all(rs <= (1e-5 if dtype == "fp32" else 2e-2) * np.abs(g).max() + 1e-12)


def test_label_gather_is_exact(hk, cuda):
    """Rows built so that loss is exactly representable: a zero logit at one
    position (the maximum), -8192 elsewhere and -2^(r+4) under the label; every
    other exponential vanishes next to exp(0) at the precision of the result."""
    import torch
    cols = 32000
    labs = np.array([0, 1, 7, 8, 255, 4095, 31999, 16000, 12345], dtype=np.int64)
    rows = len(labs)
    for dtype, tdt in (("bf16", torch.bfloat16), ("fp32", torch.float32)):
        x = np.full((rows, cols), -8192.0, dtype=np.float32)
        for r in range(rows):
            x[r, (int(labs[r]) + 3) % cols] = 0.0        # the row maximum
            x[r, labs[r]] = -float(2 ** (r + 4))         # distinct value under the label
        tx = helpers.to_torch(x, dtype, cuda)
        tl = torch.from_numpy(labs).to(cuda)
        tloss = torch.empty(rows, dtype=tdt, device=cuda)
        hk.sce_sparse_fwd(tx, tl, tloss, IGN)
        torch.cuda.synchronize()
        got = tloss.float().cpu().numpy()
        assert np.array_equal(got, np.array([float(2 ** (r + 4)) for r in range(rows)], dtype=np.float32))


def test_out_of_range_label_is_nan(hk, cuda):
    import torch
    x = helpers.to_torch(helpers.draw(1, (3, 64)), "fp32", cuda)
    tl = torch.tensor([5, 64, -3], dtype=torch.int64, device=cuda)
    loss = torch.empty(3, device=cuda)
    hk.sce_sparse_fwd(x, tl, loss, IGN)
    torch.cuda.synchronize()
    v = loss.cpu().numpy()
    assert np.isfinite(v[0]) and np.isnan(v[1]) and np.isnan(v[2])


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(9, 64), (33, 1000), (6, 32000), (5, 7)])
def test_sce_dense(hk, cuda, dtype, shape):
    import torch
    rows, cols = shape
    x = helpers.draw(601, shape, "normal", 0.0, 2.0, dtype)
    lab = helpers.rng(602).random(shape, dtype=np.float32)
    lab = oracle.round_to(lab / lab.sum(1, keepdims=True), dtype)
    eloss = oracle.sce_dense_fwd(x, lab)
    tx, tl = helpers.to_torch(x, dtype, cuda), helpers.to_torch(lab, dtype, cuda)
    tloss = torch.empty(rows, dtype=tx.dtype, device=cuda)
    hk.sce_dense_fwd(tx, tl, tloss)
    torch.cuda.synchronize()
    helpers.assert_close(tloss, eloss, dtype, "loss")
    g = helpers.draw(603, (rows,), "uniform", 0.5, 1.5, dtype)
    edx = oracle.sce_dense_bwd(x, lab, g)
    tg = helpers.to_torch(g, dtype, cuda)
    tdx = torch.empty_like(tx)
    hk.sce_dense_bwd(tx, tl, tg, tdx)
    torch.cuda.synchronize()
    helpers.assert_close(tdx, edx, dtype, "dlogits")


def test_sce_full_size_bf16(hk, cuda):
    """[16384, 32000] bf16, 5 % ignored labels, mean reduction over ALL rows."""
    import torch
    rows, cols = 16384, 32000
    g = torch.Generator(device="cpu").manual_seed(501)
    tx = (torch.randn((rows, cols), generator=g, dtype=torch.float32) * 2.0).to(torch.bfloat16).to(cuda)
    lab = _labels(rows, cols, 502, 0.05)
    tl = torch.from_numpy(lab).to(cuda)
    tloss = torch.empty(rows, dtype=torch.bfloat16, device=cuda)
    hk.sce_sparse_fwd(tx, tl, tloss, IGN)
    tg = torch.full((rows,), 1.0 / rows, dtype=torch.bfloat16, device=cuda)
    tdx = torch.empty_like(tx)
    hk.sce_sparse_bwd(tx, tl, tg, tdx, IGN)
    torch.cuda.synchronize()
    sel = np.unique(np.append(helpers.sample_rows(4, rows, 24), int(np.nonzero(lab == IGN)[0][0])))
    xs = helpers.to_numpy(tx[torch.from_numpy(sel).to(cuda)])
    eloss = oracle.sce_sparse_fwd(xs, lab[sel], IGN)
    helpers.assert_close(tloss[torch.from_numpy(sel).to(cuda)], eloss, "bf16", "loss")
    edx = oracle.sce_sparse_bwd(xs, lab[sel], np.full(len(sel), helpers.to_numpy(tg[:1])[0]), IGN)
    helpers.assert_close(tdx[torch.from_numpy(sel).to(cuda)], edx, "bf16", "dlogits")
    ign = torch.from_numpy(lab == IGN).to(cuda)
    assert torch.count_nonzero(tloss[ign]) == 0
    assert torch.count_nonzero(tdx[ign]) == 0
    # the op's mean divides by ALL rows, ignored ones included
    mean_all = tloss.float().sum().item() / rows
    n_valid = int((lab != IGN).sum())
    assert abs(mean_all - tloss.float()[~ign].mean().item() * n_valid / rows) <= 1e-4


def test_large_common_offset(hk, cuda):
    """Logits around +1000 / -3000 in fp32: the shift must cancel exactly, no precision is lost."""
    import torch
    for shift in (1000.0, -3000.0):
        x = (helpers.draw(77, (16, 4096), "normal", 0.0, 2.0) + np.float32(shift)).astype(np.float32)
        lab = _labels(16, 4096, 78, 0.0)
        tx, tl = helpers.to_torch(x, "fp32", cuda), torch.from_numpy(lab).to(cuda)
        tloss = torch.empty(16, device=cuda)
        hk.sce_sparse_fwd(tx, tl, tloss, IGN)
        g = np.full(16, 1.0, dtype=np.float32)
        tdx = torch.empty_like(tx)
        hk.sce_sparse_bwd(tx, tl, helpers.to_torch(g, "fp32", cuda), tdx, IGN)
        torch.cuda.synchronize()
        helpers.assert_close(tloss, oracle.sce_sparse_fwd(x, lab, IGN), "fp32", "loss")
        edx = oracle.sce_sparse_bwd(x, lab, g, IGN)
        helpers.assert_close(tdx, edx, "fp32", "dlogits")
