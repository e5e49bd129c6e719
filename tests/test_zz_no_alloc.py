"""hk_dropout_add_ln_bwd_static, the entry point that allocates nothing: its results equal those of
hk_dropout_add_ln_bwd (caller workspace) bit for bit, on two calls in a row that share the library's
static scratch, the second on a smaller input; shapes whose partials do not fit are refused."""
import ctypes

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu


def _inputs(rows, cols, dt, dev, seed):
    x = helpers.to_torch(helpers.draw(seed, (rows, cols), dtype=dt), dt, dev)
    dz = helpers.to_torch(helpers.draw(seed + 1, (rows, cols), dtype=dt), dt, dev)
    w = helpers.to_torch(helpers.draw(seed + 2, (cols,), "uniform", 0.8, 1.2, dt), dt, dev)
    return x, dz, w


def _both(hk, rows, cols, dt, dev, seed, is_rms, with_residual_grad):
    import torch
    x, dz, w = _inputs(rows, cols, dt, dev, seed)
    mu = torch.empty(rows, device=dev)
    rs = torch.empty(rows, device=dev)
    z = torch.empty_like(x)
    hk.dropout_add_ln_fwd(x, None, w, None, z, None, mu, rs, 1e-6, is_rms)
    dx_in = helpers.to_torch(helpers.draw(seed + 3, (rows, cols), dtype=dt), dt, dev) if with_residual_grad else None
    out = []
    for fn in (hk.dropout_add_ln_bwd, hk.dropout_add_ln_bwd_static):
        dx = torch.full_like(x, float("nan"))
        dres = torch.full_like(x, float("nan")) if with_residual_grad else None
        dg = torch.full_like(w, float("nan"))
        db = torch.full_like(w, float("nan"))
        fn(dz, dx_in, x, mu, rs, w, dx, dres, dg, db, is_rms)
        torch.cuda.synchronize()
        out.append((dx, dres, dg, db))
    return out


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_static_scratch_matches_the_workspace_call_twice(hk, cuda, dt):
    import torch
    # first call fills more of the scratch than the second uses: stale partials of the larger call
    # must not enter the smaller one's column sums
    for rows, cols, is_rms, res in ((4096, 4096, True, False), (301, 1024, False, True), (7, 264, True, False)):
        ref, got = _both(hk, rows, cols, dt, cuda, 900 + rows, is_rms, res)
        for name, a, b in zip(("dx0", "dresidual", "dgamma", "dbeta"), ref, got):
            if a is None:
                continue
            assert not torch.isnan(b.float()).any(), "%s has unwritten elements (%d x %d)" % (name, rows, cols)
            assert torch.equal(a, b), "%s differs between the workspace and the static call (%d x %d)" % (name, rows, cols)


def test_static_scratch_matches_the_oracle(hk, cuda):
    import torch
    import oracle
    rows, cols, dt = 512, 4096, "bf16"
    x = helpers.draw(402, (rows, cols), dtype=dt)
    w = helpers.draw(403, (cols,), "uniform", 0.8, 1.2, dt)
    dz = helpers.draw(404, (rows, cols), dtype=dt)
    tx, tw, tdz = (helpers.to_torch(v, dt, cuda) for v in (x, w, dz))
    mu, rs, z = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda), torch.empty_like(tx)
    hk.dropout_add_ln_fwd(tx, None, tw, None, z, None, mu, rs, 1e-6, True)
    dx, dg, db = torch.empty_like(tx), torch.empty_like(tw), torch.empty_like(tw)
    hk.dropout_add_ln_bwd_static(tdz, None, tx, mu, rs, tw, dx, None, dg, db, True)
    torch.cuda.synchronize()
    edx, edg, edb = oracle.dropout_add_ln_bwd(dz, None, x, helpers.to_numpy(mu), helpers.to_numpy(rs), w, True)
    helpers.assert_close(dx, edx, dt, "dx0")
    helpers.assert_close(dg, edg, dt, "dgamma")
    helpers.assert_close(db, edb, dt, "dbeta")


def test_static_scratch_refuses_what_does_not_fit(hk, cuda):
    import torch
    # 8192 bf16 columns on 256 persistent workgroups need exactly the 16 MiB the scratch holds; a plan with
    # more workgroups (forced here through the launch-shape override) needs more and must be refused
    rows, cols = 2048, 8192
    x = torch.zeros(rows, cols, device=cuda, dtype=torch.bfloat16)
    w = torch.ones(cols, device=cuda, dtype=torch.bfloat16)
    st = torch.ones(rows, device=cuda)
    dx, dg, db = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    hk.tune_set("norm_bwd_blocks", 512)
    try:
        need = hk.norm_bwd_workspace_bytes(hk.DTYPES["bf16"], rows, cols)
        assert need > (16 << 20)
        with pytest.raises(hk.HkError) as e:
            hk.dropout_add_ln_bwd_static(x, None, x, st, st, w, dx, None, dg, db, True)
        assert e.value.code == -4 and "static scratch" in str(e.value)
    finally:
        hk.tune_set("norm_bwd_blocks", 0)
    # the automatic plan of the same shape fits, and runs
    assert hk.norm_bwd_workspace_bytes(hk.DTYPES["bf16"], rows, cols) <= (16 << 20)
    hk.dropout_add_ln_bwd_static(x, None, x, st, st, w, dx, None, dg, db, True)
    torch.cuda.synchronize()
    assert float(dx.float().abs().max()) == 0.0


def test_static_scratch_allocates_nothing(hk, cuda):
    """The property the entry point exists for: after the first call on the device (which looks the scratch's
    address up), repeated calls leave the device's free memory where it was, through the driver's own count and
    through torch's caching allocator, and the library's device pool, neither of which is asked for a byte."""
    import torch
    rows, cols, dt = 1024, 4096, "bf16"
    x, dz, w = _inputs(rows, cols, dt, cuda, 77)
    mu, rs, z = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda), torch.empty_like(x)
    hk.dropout_add_ln_fwd(x, None, w, None, z, None, mu, rs, 1e-6, True)
    dx, dg, db = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    hk.dropout_add_ln_bwd_static(dz, None, x, mu, rs, w, dx, None, dg, db, True)      # first call on the device
    torch.cuda.synchronize()
    free0 = ctypes.c_size_t()
    total = ctypes.c_size_t()
    hk.check(hk.lib().hk_mem_get_info(ctypes.byref(free0), ctypes.byref(total)))
    stats0 = torch.cuda.memory_stats()
    for _ in range(20):
        hk.dropout_add_ln_bwd_static(dz, None, x, mu, rs, w, dx, None, dg, db, True)
    torch.cuda.synchronize()
    free1 = ctypes.c_size_t()
    hk.check(hk.lib().hk_mem_get_info(ctypes.byref(free1), ctypes.byref(total)))
    stats1 = torch.cuda.memory_stats()
    assert free1.value == free0.value, "device free memory moved across static calls"
    for key in ("allocation.all.allocated", "segment.all.allocated", "num_alloc_retries"):
        assert stats1.get(key, 0) == stats0.get(key, 0), key


def test_static_scratch_under_graph_capture(hk, cuda):
    """Recorded into a HIP graph after a first call outside the capture (the address look-up of the scratch is
    made once per device and not again), the static call replays: every replay, with new inputs written in place
    and eager work and synchronisations between replays, equals the eager workspace call bit for bit."""
    import torch
    rows, cols, bf = 768, 4096, torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(rows, cols, generator=g, device=cuda).to(bf)
    dz = torch.randn(rows, cols, generator=g, device=cuda).to(bf)
    w = (torch.rand(cols, generator=g, device=cuda) * 0.4 + 0.8).to(bf)
    mu, rs, z = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda), torch.empty_like(x)
    dx, dg, db = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(hk.norm_bwd_workspace_bytes(hk.dtype_code(x), rows, cols) // 4 + 4, device=cuda)

    def step():
        hk.dropout_add_ln_fwd(x, None, w, None, z, None, mu, rs, 1e-6, True)
        hk.dropout_add_ln_bwd_static(dz, None, x, mu, rs, w, dx, None, dg, db, True)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                      # first call on the device, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for trial in range(4):
        x.copy_(torch.randn(rows, cols, generator=g, device=cuda).to(bf))
        dz.copy_(torch.randn(rows, cols, generator=g, device=cuda).to(bf))
        # eager reference through the workspace call
        edx, edg, edb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
        emu, ers, ez = torch.empty_like(mu), torch.empty_like(rs), torch.empty_like(z)
        hk.dropout_add_ln_fwd(x, None, w, None, ez, None, emu, ers, 1e-6, True)
        hk.dropout_add_ln_bwd(dz, None, x, emu, ers, w, edx, None, edg, edb, True, workspace=ws)
        torch.cuda.synchronize()
        for t in (dx, dg, db):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dx, edx) and torch.equal(dg, edg) and torch.equal(db, edb), "replay %d" % trial
