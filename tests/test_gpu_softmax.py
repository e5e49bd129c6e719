"""GPU parity of Softmax forward / backward against the oracle (hk_softmax_*)."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape,dim", [((7, 64), -1), ((3, 5, 2048), -1), ((33, 1000), 1), ((4, 7), -1),
                                       ((2, 3, 4096), 2), ((2, 20000), -1), ((1, 70000), -1),
                                       ((4, 6, 10), 1), ((5, 33, 7, 3), 1), ((16, 8), 0)])
def test_softmax_fwd_bwd(hk, cuda, dtype, shape, dim):
    import torch
    x = helpers.draw(201, shape, "normal", 0.0, 3.0, dtype)
    ey = oracle.softmax_fwd(x, dim)
    tx = helpers.to_torch(x, dtype, cuda)
    ty = torch.empty_like(tx)
    hk.softmax_fwd(tx, ty, dim)
    torch.cuda.synchronize()
    helpers.assert_close(ty, ey, dtype, "y")
    sums = ty.float().sum(dim % len(shape)).cpu().numpy()
    assert np.max(np.abs(sums - 1.0)) <= (2e-2 if dtype != "fp32" else 1e-5)

    y = helpers.to_numpy(ty)                      # backward consumes the stored y
    dy = helpers.draw(202, shape, dtype=dtype)
    edx = oracle.softmax_bwd(y, dy, dim)
    tdy = helpers.to_torch(dy, dtype, cuda)
    tdx = torch.empty_like(tx)
    hk.softmax_bwd(ty, tdy, tdx, dim)
    torch.cuda.synchronize()
    helpers.assert_close(tdx, edx, dtype, "dx", ordinary_rtol=helpers.SOFTMAX_GRADIENT_ORDINARY_RTOL)


def test_softmax_special_rows(hk, cuda):
    import torch
    cols = 2048
    x = np.zeros((4, cols), dtype=np.float32)
    x[0, :] = 5.0                       # all equal -> uniform
    x[1, :] = -np.inf; x[1, 17] = 0.0   # one finite logit -> one-hot
    x[2, :] = -80.0; x[2, 5] = 80.0     # dominant logit
    x[3, :] = helpers.draw(9, (cols,)) + 1000.0   # large common offset
    tx = helpers.to_torch(x, "fp32", cuda)
    ty = torch.empty_like(tx)
    hk.softmax_fwd(tx, ty)
    torch.cuda.synchronize()
    y = ty.cpu().numpy()
    assert np.allclose(y[0], 1.0 / cols, rtol=1e-6)
    assert y[1, 17] == 1.0 and y[1].sum() == 1.0
    assert y[2, 5] == 1.0 and y[2].sum() == 1.0
    ref = oracle.softmax_fwd(x[3][None, :])[0]
    assert np.max(np.abs(y[3] - ref)) <= 1e-5 * ref.max()


def test_softmax_full_size_bf16(hk, cuda):
    """[4, 32, 2048, 2048] bf16: GPU on everything, oracle on sampled rows."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(201)
    shape = (4, 32, 2048, 2048)
    tx = (torch.randn(shape, generator=g, dtype=torch.float32) * 3.0).to(torch.bfloat16).to(cuda)
    ty = torch.empty_like(tx)
    hk.softmax_fwd(tx, ty)
    tdy = torch.randn(shape, generator=g, dtype=torch.float32).to(torch.bfloat16).to(cuda)
    tdx = torch.empty_like(tx)
    hk.softmax_bwd(ty, tdy, tdx)
    torch.cuda.synchronize()
    rows = 4 * 32 * 2048
    sel = torch.from_numpy(helpers.sample_rows(3, rows, 64)).to(cuda)
    x2, y2, dy2, dx2 = (t.view(rows, 2048)[sel] for t in (tx, ty, tdy, tdx))
    ey = oracle.softmax_fwd(helpers.to_numpy(x2))
    helpers.assert_close(y2, ey, "bf16", "y")
    edx = oracle.softmax_bwd(helpers.to_numpy(y2), helpers.to_numpy(dy2))
    helpers.assert_close(dx2, edx, "bf16", "dx")
    # size-independent properties on the whole tensor
    s = ty.view(rows, 2048).float().sum(1)
    assert float((s - 1).abs().max()) <= 2e-2
    assert float(tdx.view(rows, 2048).float().sum(1).abs().max()) <= 5e-2
