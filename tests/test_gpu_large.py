"""Arrays of more than 2^31 elements: every index computation past the 32-bit range.  The inputs are drawn on the
GPU; the kernels run on the whole array; the oracle checks a sample of rows (rows are independent) that holds the
first rows, the rows on either side of element 2^31 and the last rows, and column results are checked against
float64 sums taken in slices."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

COLS = 2048
ROWS = (1 << 20) + 5                      # 2^31 + 10240 elements
EDGE = (1 << 31) // COLS                  # the row that starts at element 2^31


def _sample(rows, edge):
    return np.array([0, 1, 2, edge - 1, edge, edge + 1, rows - 2, rows - 1])


def _randn(torch, shape, seed, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda", dtype=torch.bfloat16) * scale


def _column_sums(torch, fn, rows, step=1 << 16):
    """float64 sum over rows of fn(lo, hi) -> [hi - lo, cols] float64, in slices."""
    total = None
    for lo in range(0, rows, step):
        part = fn(lo, min(rows, lo + step)).sum(0)
        total = part if total is None else total + part
    return total.cpu().numpy()


def test_rmsnorm_forward_backward_past_2_31_elements(hk, cuda):
    import torch
    x, dz = _randn(torch, (ROWS, COLS), 1), _randn(torch, (ROWS, COLS), 2)
    w = (torch.rand(COLS, device=cuda) * 0.4 + 0.8).to(torch.bfloat16)
    z, dx = torch.empty_like(x), torch.empty_like(x)
    mu, rs = torch.empty(ROWS, device=cuda), torch.empty(ROWS, device=cuda)
    dg, db = torch.empty_like(w), torch.empty_like(w)
    hk.dropout_add_ln_fwd(x, None, w, None, z, None, mu, rs, 1e-6, True)
    hk.dropout_add_ln_bwd(dz, None, x, mu, rs, w, dx, None, dg, db, True)
    torch.cuda.synchronize()
    sel = _sample(ROWS, EDGE)
    xs, dzs, ws = helpers.to_numpy(x[sel]), helpers.to_numpy(dz[sel]), helpers.to_numpy(w)
    ez, _, _, ers = oracle.dropout_add_ln_fwd(xs, None, ws, None, 1e-6, True)
    helpers.assert_close(z[sel], ez, "bf16", "z")
    helpers.assert_close(rs[sel], ers, "fp32", "rsigma")
    rs_sel = helpers.to_numpy(rs[sel])
    edx, _, _ = oracle.dropout_add_ln_bwd(dzs, None, xs, np.zeros(len(sel)), rs_sel, ws, True)
    helpers.assert_close(dx[sel], edx, "bf16", "dx")
    want = _column_sums(torch, lambda lo, hi: dz[lo:hi].double() * x[lo:hi].double() * rs[lo:hi].double()[:, None],
                        ROWS)
    helpers.assert_close(dg, want, "bf16", "dgamma over 2^20 rows")
    helpers.assert_close(db, _column_sums(torch, lambda lo, hi: dz[lo:hi].double(), ROWS), "bf16", "dbeta")


def test_softmax_past_2_31_elements(hk, cuda):
    import torch
    x, dy = _randn(torch, (ROWS, COLS), 3, 2.0), _randn(torch, (ROWS, COLS), 4)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    hk.softmax_fwd(x, y, -1)
    hk.softmax_bwd(y, dy, dx, -1)
    torch.cuda.synchronize()
    sel = _sample(ROWS, EDGE)
    helpers.assert_close(y[sel], oracle.softmax_fwd(helpers.to_numpy(x[sel])), "bf16", "softmax")
    helpers.assert_close(dx[sel], oracle.softmax_bwd(helpers.to_numpy(y[sel]), helpers.to_numpy(dy[sel])), "bf16",
                         "softmax gradient")


def test_cross_entropy_past_2_31_elements(hk, cuda):
    import torch
    rows, cols = 67110, 32000              # 2 147 520 000 elements
    edge = (1 << 31) // cols
    x = _randn(torch, (rows, cols), 5, 2.0)
    labels = torch.randint(0, cols, (rows,), device=cuda)
    labels[::11] = -100
    loss = torch.empty(rows, dtype=torch.bfloat16, device=cuda)
    grad = _randn(torch, (rows,), 6)
    dx = torch.empty_like(x)
    hk.sce_sparse_fwd(x, labels, loss, -100)
    hk.sce_sparse_bwd(x, labels, grad, dx, -100)
    torch.cuda.synchronize()
    sel = _sample(rows, edge)
    xs, ls = helpers.to_numpy(x[sel]), labels[sel].cpu().numpy()
    helpers.assert_close(loss[sel], oracle.sce_sparse_fwd(xs, ls, -100), "bf16", "loss")
    helpers.assert_close(dx[sel], oracle.sce_sparse_bwd(xs, ls, helpers.to_numpy(grad[sel]), -100), "bf16", "dlogits")
    # every row of the gradient sums to zero (softmax sums to one, minus the one-hot), ignored rows are zero
    row_sums = torch.stack([dx[lo:lo + 4096].float().sum(1).abs().max() for lo in range(0, rows, 4096)]).max().item()
    assert row_sums <= 0.05
    assert (dx[::11] == 0).all()


def test_elementwise_and_broadcast_past_2_31_elements(hk, cuda):
    import torch
    x = _randn(torch, (ROWS, COLS), 7)
    per_row = _randn(torch, (ROWS, 1), 8)
    out = torch.empty_like(x)
    sel = _sample(ROWS, EDGE)
    hk.binary("sub", x, per_row, out)
    torch.cuda.synchronize()
    want = helpers.to_numpy(x[sel]).astype(np.float64) - helpers.to_numpy(per_row[sel]).astype(np.float64)
    helpers.assert_close(out[sel], want, "bf16", "x - per-row value")
    hk.unary("exp", x, out)
    torch.cuda.synchronize()
    helpers.assert_close(out[sel], np.exp(helpers.to_numpy(x[sel]).astype(np.float64)), "bf16", "exp")
    hk.broadcast(per_row, out, scalar=0.5)
    torch.cuda.synchronize()
    assert torch.equal(out[sel], (per_row[sel] * 0.5).expand(len(sel), COLS))
    assert torch.equal(out[:, COLS - 1], (per_row[:, 0] * 0.5))          # the last column of every row


def test_reduce_past_2_31_elements(hk, cuda):
    import torch
    x = _randn(torch, (ROWS, COLS), 9)
    rows_out = torch.empty(ROWS, dtype=torch.bfloat16, device=cuda)
    cols_out = torch.empty(COLS, dtype=torch.bfloat16, device=cuda)
    hk.reduce(x, rows_out, [1], "sum")
    hk.reduce(x, cols_out, [0], "mean")
    torch.cuda.synchronize()
    sel = _sample(ROWS, EDGE)
    helpers.assert_close(rows_out[sel], helpers.to_numpy(x[sel]).astype(np.float64).sum(1), "bf16", "row sums")
    want = _column_sums(torch, lambda lo, hi: x[lo:hi].double(), ROWS) / ROWS
    # a mean of 2^20 standard normal draws is ~1e-3: compare on the scale of one draw's share
    helpers.assert_close(cols_out, want, "bf16", "column means", scale=1e-3)
    nrm = torch.empty(ROWS, dtype=torch.bfloat16, device=cuda)
    hk.norm(x, nrm, 1, 2)
    torch.cuda.synchronize()
    helpers.assert_close(nrm[sel], np.sqrt((helpers.to_numpy(x[sel]).astype(np.float64) ** 2).sum(1)), "bf16", "2-norm")


def test_batch_norm_past_2_31_elements(hk, cuda):
    import torch
    n, c, hw = 33, 64, 1024 * 1024 + 8       # 2 214 609 920 elements
    x = _randn(torch, (n, c, hw), 10, 1.5) + 0.25
    y = torch.empty_like(x)
    scale, bias = torch.rand(c, device=cuda) + 0.5, torch.randn(c, device=cuda)
    rm, rv = torch.zeros(c, device=cuda), torch.ones(c, device=cuda)
    sm, si = torch.empty(c, device=cuda), torch.empty(c, device=cuda)
    hk.batch_norm_fwd(x, scale, bias, y, 0.1, 1e-5, rm, rv, sm, si)
    torch.cuda.synchronize()
    mean = torch.stack([x[:, ch].double().mean() for ch in range(c)])
    var = torch.stack([((x[:, ch].double() - mean[ch]) ** 2).mean() for ch in range(c)])
    helpers.assert_close(sm, mean.cpu().numpy(), "fp32", "saved mean", scale=1.0)
    helpers.assert_close(si, (1.0 / torch.sqrt(var + 1e-5)).cpu().numpy(), "fp32", "saved inverse deviation")
    for img, ch in ((0, 0), (15, 31), (16, 0), (32, 63)):       # image 15/16: either side of element 2^31
        want = (x[img, ch].double() - mean[ch]) / torch.sqrt(var[ch] + 1e-5) * scale[ch].double() + bias[ch].double()
        got = y[img, ch].double()
        assert ((got - want).abs() <= 1e-2 * (want.abs() + 1.0)).all()
