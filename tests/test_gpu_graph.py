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


def test_graph_replays_match_eager_widened_calls(hk, cuda):
    """The same for the calls around the core path: dropout + residual + norm block, batch norm, element-wise
    and broadcast kernels, p-norm, the fused vocabulary-parallel loss and the reduced-loss gradient."""
    import torch
    rows, cols, vocab = 256, 2048, 4096
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(21)

    def randn(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g, device=cuda) * scale).to(bf)

    x0, res, dz = randn(rows, cols), randn(rows, cols), randn(rows, cols)
    w = (torch.rand(cols, generator=g, device=cuda) * 0.4 + 0.8).to(bf)
    z, xsum, dx0, dres = (torch.empty(rows, cols, dtype=bf, device=cuda) for _ in range(4))
    dmask = torch.empty(rows, cols, dtype=torch.uint8, device=cuda)
    mu, rs = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    dg = torch.empty(cols, dtype=bf, device=cuda)
    img, dimg = randn(8, 16, 12, 12, scale=2.0), randn(8, 16, 12, 12)
    bn_y, bn_dx = torch.empty_like(img), torch.empty_like(img)
    bn_scale = torch.rand(16, generator=g, device=cuda) + 0.5
    bn_bias = torch.randn(16, generator=g, device=cuda)
    run_mean, run_var = torch.zeros(16, device=cuda), torch.ones(16, device=cuda)
    sv_mean, sv_inv, bn_ds, bn_db = (torch.empty(16, device=cuda) for _ in range(4))
    logits = randn(rows, vocab, scale=2.0)
    labels = torch.randint(0, vocab, (rows,), generator=g, device=cuda)
    labels[::7] = -100
    row_max = torch.empty(rows, 1, dtype=bf, device=cuda)
    shifted, expd, dlogits, dfused = (torch.empty_like(logits) for _ in range(4))
    stats = torch.empty(3, rows, device=cuda)
    loss, nrm = torch.empty(rows, dtype=bf, device=cuda), torch.empty(rows, dtype=bf, device=cuda)
    lse = torch.empty(rows, device=cuda)
    grad_out = torch.full((1,), 0.5, dtype=bf, device=cuda)
    back = torch.empty(rows, cols, dtype=bf, device=cuda)
    dnorm = torch.empty(rows, cols, dtype=bf, device=cuda)
    hk.dropout_add_ln_fwd_ex(x0, w, z, mu, rs, residual=res, x=xsum, dmask=dmask, dropout_p=0.1, eps=1e-6,
                             is_rms=True, seed=1234, offset=8)
    ws_dal = hk.dropout_add_ln_bwd_ex(dz, xsum, mu, rs, w, dx0, dmask=dmask, dresidual=dres, dgamma=dg,
                                      dropout_p=0.1, is_rms=True)      # allocates and returns its workspace
    ws_bn = torch.empty(hk.batch_norm_workspace_bytes(img) // 4 + 4, device=cuda)
    ws_max = torch.empty(max(1, hk.reduce_workspace_bytes(8, [rows, vocab], [vocab, 1], [1]) // 4 + 4), device=cuda)
    ws_nrm = torch.empty(max(1, hk.reduce_workspace_bytes(8, [rows, cols], [cols, 1], [1]) // 4 + 4), device=cuda)

    def step():
        hk.dropout_add_ln_fwd_ex(x0, w, z, mu, rs, residual=res, x=xsum, dmask=dmask, dropout_p=0.1, eps=1e-6,
                                 is_rms=True, seed=1234, offset=8)
        hk.dropout_add_ln_bwd_ex(dz, xsum, mu, rs, w, dx0, dmask=dmask, dresidual=dres, dgamma=dg, dropout_p=0.1,
                                 is_rms=True, workspace=ws_dal)
        hk.batch_norm_fwd(img, bn_scale, bn_bias, bn_y, 0.1, 1e-5, run_mean, run_var, sv_mean, sv_inv, workspace=ws_bn)
        hk.batch_norm_bwd(dimg, img, bn_scale, bn_dx, bn_ds, bn_db, sv_mean, sv_inv, workspace=ws_bn)
        hk.reduce(logits, row_max, [1], "max", workspace=ws_max)
        hk.binary("sub", logits, row_max, shifted)
        hk.unary("exp", shifted, expd)
        hk.vocab_parallel_ce_stats(logits, labels, stats, 0, -100)
        hk.vocab_parallel_ce_combine(stats.view(1, 3, rows), labels, -100, loss, lse)
        hk.vocab_parallel_ce_bwd_fused(logits, labels, lse, loss, dfused, 0, -100)
        hk.sce_sparse_bwd_reduced(logits, labels, grad_out, 1.0 / rows, dlogits, -100)
        hk.norm(xsum, nrm, 1, 2, workspace=ws_nrm)
        hk.norm_bwd(xsum, nrm, loss, dnorm, 1, 2)
        hk.broadcast(loss.view(rows, 1), back, scalar=1.0 / cols)

    outs = (z, xsum, dmask, mu, rs, dx0, dres, dg, bn_y, bn_dx, bn_ds, bn_db, sv_mean, sv_inv, row_max, shifted,
            expd, stats, loss, lse, dfused, dlogits, nrm, dnorm, back)

    def snapshot():
        torch.cuda.synchronize()
        return [o.clone() for o in outs]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for trial in range(3):
        x0.copy_(randn(rows, cols)); dz.copy_(randn(rows, cols)); img.copy_(randn(8, 16, 12, 12, scale=2.0))
        logits.copy_(randn(rows, vocab, scale=2.0))
        run_mean.zero_(); run_var.fill_(1.0)          # the running statistics are updated in place by every call
        step()
        want = snapshot()
        want_running = (run_mean.clone(), run_var.clone())
        for o in outs:
            o.fill_(float("nan")) if o.is_floating_point() else o.zero_()
        run_mean.zero_(); run_var.fill_(1.0)
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "output %d differs on replay %d" % (i, trial)
        assert torch.equal(run_mean, want_running[0]) and torch.equal(run_var, want_running[1])


def test_graph_replays_of_the_large_input_forward_launches(hk, cuda):
    """Inputs tall enough for the forward norm's two-rows-per-workgroup launch (which asks for dynamic LDS to bound
    the workgroups resident per compute unit) recorded into a graph: RMSNorm at 4096 bf16 columns (256 threads),
    LayerNorm at 4096 fp32 columns (512 threads) and at 5120 bf16 columns (320 threads); every replay equals eager."""
    import torch
    g = torch.Generator(device=cuda).manual_seed(778)
    bf = torch.bfloat16
    rows = 8192
    cases = []
    for cols, dt, rms in ((4096, bf, True), (4096, torch.float32, False), (5120, bf, False)):
        x = torch.randn(rows, cols, generator=g, device=cuda).to(dt)
        w = (torch.rand(cols, generator=g, device=cuda) + 0.5).to(dt)
        b = None if rms else (torch.randn(cols, generator=g, device=cuda) * 0.1).to(dt)
        y = torch.empty_like(x)
        mu, rs = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
        cases.append((x, w, b, y, mu, rs, rms))

    def step():
        for x, w, b, y, mu, rs, rms in cases:
            if rms:
                hk.dropout_add_ln_fwd(x, None, w, None, y, None, mu, rs, 1e-6, True)
            else:
                hk.layer_norm_fwd(x, w, b, y, mu, rs, 1e-5, stat_kind=1)

    outs = [t for c in cases for t in (c[3], c[4], c[5])]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for trial in range(3):
        for c in cases:
            c[0].copy_(torch.randn(c[0].shape, generator=g, device=cuda).to(c[0].dtype))
        step()
        torch.cuda.synchronize()
        want = [o.clone() for o in outs]
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(outs, want)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "output %d differs on replay %d" % (i, trial)
