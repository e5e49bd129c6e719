"""GPU parity of the negative log-likelihood loss (hk_nll_loss_fwd / _bwd and NLLLossCuda /
NLLLossGradientCuda): a gather and a fill-with-scatter, so every comparison is exact."""
import importlib

import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16", "fp64"])
@pytest.mark.parametrize("shape", [(37, 1000), (5, 7), (64, 32000), (1, 8), (300, 33)])
def test_nll_loss_is_exact(hk, cuda, dtype, shape):
    import torch
    rows, cols = shape
    pred = helpers.draw(1 + cols, shape, dtype=dtype if dtype != "fp64" else "fp32")
    labels = helpers.rng(2 + cols).integers(0, cols, size=rows).astype(np.int64)
    labels[::5] = -100
    if rows > 3:
        labels[3] = cols          # just past the end
    gl = helpers.draw(3 + cols, (rows,), dtype=dtype if dtype != "fp64" else "fp32")
    tp, tg = helpers.to_torch(pred, dtype, cuda), helpers.to_torch(gl, dtype, cuda)
    tl = torch.from_numpy(labels).to(cuda)
    tloss = torch.full((rows,), 7.0, dtype=tp.dtype, device=cuda)
    tout = torch.full(shape, 7.0, dtype=tp.dtype, device=cuda)
    hk.nll_loss_fwd(tp, tl, tloss)
    hk.nll_loss_bwd(tl, tg, tout)
    torch.cuda.synchronize()
    assert np.array_equal(helpers.to_numpy(tloss).astype(np.float64), oracle.nll_loss_fwd(pred, labels))
    want = oracle.nll_loss_bwd(labels, gl, cols)
    want = oracle.round_to(want.astype(np.float32), dtype).astype(np.float64) if dtype != "fp64" else want
    assert np.array_equal(helpers.to_numpy(tout).astype(np.float64), want)


def test_nll_loss_through_the_operator_layer(hk, cuda):
    import torch
    ops = importlib.import_module("hotspa-ae_amd.hetu_ops")
    shape = (4, 9, 512)
    pred = helpers.draw(11, shape, dtype="bf16")
    labels = helpers.rng(12).integers(0, 512, size=shape[:-1]).astype(np.int64)
    gl = helpers.draw(13, shape[:-1], dtype="bf16")
    tp, tg = helpers.to_torch(pred, "bf16", cuda), helpers.to_torch(gl, "bf16", cuda)
    tl = torch.from_numpy(labels).to(cuda)
    tloss = torch.empty(shape[:-1], dtype=tp.dtype, device=cuda)
    tout = torch.empty_like(tp)
    torch.cuda.synchronize()
    ops.nll_loss(tp, tl, tloss)
    ops.nll_loss_gradient(tp, tl, tg, tout)
    ops.stream_sync()
    assert np.array_equal(helpers.to_numpy(tloss).reshape(-1).astype(np.float64),
                          oracle.nll_loss_fwd(pred.reshape(36, 512), labels.reshape(36)))
    want = oracle.round_to(oracle.nll_loss_bwd(labels.reshape(36), gl.reshape(36), 512).astype(np.float32), "bf16")
    assert np.array_equal(helpers.to_numpy(tout).reshape(36, 512), want)
    with pytest.raises(ops.AssertionError_, match="int64"):
        ops.nll_loss(tp, tl.int(), tloss)
    with pytest.raises(ops.AssertionError_):
        ops.nll_loss(tp, tl[:, :4].contiguous(), tloss)
