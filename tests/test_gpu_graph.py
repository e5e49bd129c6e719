"""The operator calls can be recorded into a HIP graph: they allocate nothing, clear nothing with
memset nodes and synchronise nothing.  Every replay is checked against the eager result, with eager
work and synchronisations between replays."""
import pytest

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager(hk, cuda):
    import torch
    rows, cols, vocab = 512, 4096, 8192
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(rows, cols, generator=g, device=cuda).to(bf)
    dz = torch.randn(rows, cols, generator=g, device=cuda).to(bf)
    w = (torch.rand(cols, generator=g, device=cuda) * 0.4 + 0.8).to(bf)
    logits = (torch.randn(rows, vocab, generator=g, device=cuda) * 2).to(bf)
    labels = torch.randint(0, vocab, (rows,), generator=g, device=cuda)
    labels[::9] = -100
    z, dx = torch.empty_like(x), torch.empty_like(x)
    mu = torch.empty(rows, device=cuda)
    rs = torch.empty(rows, device=cuda)
    dg, db = torch.empty_like(w), torch.empty_like(w)
    sm = torch.empty_like(logits)
    loss = torch.empty(rows, dtype=bf, device=cuda)
    mean_loss = torch.empty(1, dtype=bf, device=cuda)
    colsum = torch.empty(cols, dtype=bf, device=cuda)
    ws_bwd = torch.empty(hk.norm_bwd_workspace_bytes(hk.dtype_code(x), rows, cols) // 4 + 4, device=cuda)
    ws_r1 = torch.empty(max(1, hk.reduce_workspace_bytes(8, [rows], [1], [0]) // 4 + 4), device=cuda)
    ws_r2 = torch.empty(max(1, hk.reduce_workspace_bytes(8, [rows, cols], [cols, 1], [0]) // 4 + 4), device=cuda)

    def step():
        hk.dropout_add_ln_fwd(x, None, w, None, z, None, mu, rs, 1e-6, True)
        hk.dropout_add_ln_bwd(dz, None, x, mu, rs, w, dx, None, dg, db, True, workspace=ws_bwd)
        hk.softmax_fwd(logits, sm, -1)
        hk.sce_sparse_fwd(logits, labels, loss, -100)
        hk.reduce(loss, mean_loss, [0], "mean", workspace=ws_r1)
        hk.reduce(dx, colsum, [0], "sum", workspace=ws_r2)

    outs = (z, dx, mu, rs, dg, db, sm, loss, mean_loss, colsum)

    def snapshot():
        torch.cuda.synchronize()
        return [o.clone() for o in outs]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                      # warm-up outside the capture (first-use caches)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for trial in range(4):
        # new inputs, written in place so the recorded pointers stay valid
        x.copy_(torch.randn(rows, cols, generator=g, device=cuda).to(bf))
        dz.copy_(torch.randn(rows, cols, generator=g, device=cuda).to(bf))
        logits.copy_((torch.randn(rows, vocab, generator=g, device=cuda) * 2).to(bf))
        step()
        want = snapshot()
        for o in outs:
            o.fill_(float("nan")) if o.is_floating_point() else o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "output %d differs on replay %d" % (i, trial)
