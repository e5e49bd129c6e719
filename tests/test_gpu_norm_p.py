"""GPU parity of the p-norm over one dimension and its gradient (hk_norm / hk_norm_bwd) against the oracle.
The forward runs on the reduce planner, so the shapes cover its inner, outer and generic paths."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

CASES = [((64, 4096), 1), ((4096, 64), 0), ((32768, 256), 0), ((7, 33, 5), 1), ((6, 1000), 1), ((3, 5, 7, 16), 2),
         ((50, 1), 1), ((1, 40000), 1), ((9, 264, 8), 1)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16", "fp64"])
@pytest.mark.parametrize("shape,dim", CASES, ids=lambda v: str(v))
@pytest.mark.parametrize("p", [1, 2, 3, 6])
def test_norm_and_gradient(hk, cuda, dtype, shape, dim, p):
    import torch
    g = helpers.rng(sum(shape) + dim + p)
    x = g.standard_normal(shape)
    x = x.astype(np.float64) if dtype == "fp64" else oracle.round_to(x.astype(np.float32), dtype)
    x.reshape(-1)[::17] = 0.0
    want = oracle.norm_p_fwd(x, dim, p)
    tx = helpers.to_torch(x, dtype, cuda)
    out = torch.empty(want.shape, dtype=tx.dtype, device=cuda)
    hk.norm(tx, out, dim, p)
    torch.cuda.synchronize()
    helpers.assert_close(out, want, dtype, "norm")
    # gradient from the norm as stored
    n = helpers.to_numpy(out).astype(np.float64)
    grad = g.standard_normal(want.shape)
    grad = grad.astype(np.float64) if dtype == "fp64" else oracle.round_to(grad.astype(np.float32), dtype)
    want_g = oracle.norm_p_bwd(x, n, grad, dim, p)
    tg = helpers.to_torch(grad, dtype, cuda)
    dx = torch.empty_like(tx)
    hk.norm_bwd(tx, out, tg, dx, dim, p)
    torch.cuda.synchronize()
    helpers.assert_close(dx, want_g, dtype, "gradient")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("p", [1, 2, 3])
def test_norm_of_few_long_rows_is_split_over_workgroups(hk, cuda, dtype, p):
    """Few rows of 2^20 elements (a global gradient norm): the row is split over workgroups and the fp32
    partial sums of |x|^p are folded by a second launch, which must add them up as they are."""
    import torch
    shape = (4, 1 << 20)
    assert hk.reduce_workspace_bytes(hk.DTYPES[dtype], list(shape), [shape[1], 1], [1]) > 0   # the split path
    x = oracle.round_to(helpers.rng(77 + p).standard_normal(shape).astype(np.float32), dtype)
    want = oracle.norm_p_fwd(x, 1, p)
    tx = helpers.to_torch(x, dtype, cuda)
    out = torch.empty(4, dtype=tx.dtype, device=cuda)
    hk.norm(tx, out, 1, p)
    torch.cuda.synchronize()
    helpers.assert_close(out, want, dtype, "norm of split rows")
    ones = torch.ones(1, 1 << 20, dtype=tx.dtype, device=cuda)     # exact: (2^20)^(1/p)
    hk.norm(ones, out[:1], 1, 2)
    torch.cuda.synchronize()
    assert float(out[0]) == 1024.0


def test_norm_edge_cases(hk, cuda):
    import torch
    z = torch.zeros(5, 512, device=cuda)
    n = torch.empty(5, device=cuda)
    dx = torch.full_like(z, 7.0)
    for p in (1, 2, 3):
        hk.norm(z, n, 1, p)
        hk.norm_bwd(z, n, torch.ones(5, device=cuda), dx, 1, p)
        torch.cuda.synchronize()
        assert (n == 0).all() and (dx == 0).all()          # zero slices: norm 0, gradient 0 (never 0/0)
    x = torch.randn(6, 300, device=cuda)
    v = x.t()                                              # strided view, norm over what is now dim 0
    out = torch.empty(6, device=cuda)
    hk.norm(v, out, 0, 2)
    torch.cuda.synchronize()
    assert torch.allclose(out, torch.linalg.vector_norm(x, 2, dim=1), rtol=1e-5)
    big = torch.full((3, 4096), 1e20, device=cuda)         # |x|^2 overflows fp32: inf, as in the reference's arithmetic
    hk.norm(big, out[:3], 1, 2)
    torch.cuda.synchronize()
    assert torch.isinf(out[:3]).all()
    with pytest.raises(hk.HkError) as e:
        hk.norm(x, out, 1, 0)
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:
        hk.norm(x.long(), out.long(), 1, 2)
    assert e.value.code == -2
    e0 = torch.empty(0, 8, device=cuda)
    hk.norm(e0, torch.empty(0, device=cuda), 1, 2)
    hk.norm_bwd(e0, e0[:, 0], e0[:, 0], e0.clone(), 1, 2)
