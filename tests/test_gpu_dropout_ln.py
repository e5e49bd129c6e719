"""GPU parity of the full dropout-add-LayerNorm / RMSNorm interface (hk_dropout_add_ln_fwd_ex / _bwd_ex:
dropout, row and column scaling, row subsets, mixed types, parallel residual) against
oracle/dropout_add_ln.py.  Masks are integer work and compared bit for bit; floating outputs within
1e-5 (fp32) / 1e-2 (bf16, fp16) of the float64 oracle, in the type each output is stored in."""
import numpy as np
import pytest

import helpers
import oracle
from oracle import dropout_add_ln as dal

pytestmark = pytest.mark.gpu

# (weight, input, residual) types: the combinations the reference registers kernels for
COMBOS = [("fp32", "fp32", "fp32"), ("fp16", "fp16", "fp16"), ("bf16", "bf16", "bf16"),
          ("fp32", "fp16", "fp32"), ("fp32", "bf16", "fp32"), ("fp16", "fp16", "fp32"),
          ("bf16", "bf16", "fp32"), ("fp32", "fp16", "fp16"), ("fp32", "bf16", "bf16"),
          ("fp16", "fp32", "fp32")]
SHAPES = [(33, 256), (17, 1000), (9, 4096), (6, 5120), (5, 8192), (3, 8)]
SEED, OFFSET = 0x1234_5678_9abc_def0, 0x1_0000_0007


def _mask(numel, p, which=0):
    return dal.dropout_keep(SEED, OFFSET, numel, np.float32(1.0) - np.float32(p), which)


def _tt(a, dtype, cuda):
    return None if a is None else helpers.to_torch(a, dtype, cuda)


@pytest.mark.parametrize("combo", COMBOS, ids=lambda c: "w%s-i%s-r%s" % c)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "%dx%d" % s)
@pytest.mark.parametrize("features", ["types-only", "dropout", "scales", "all"])
@pytest.mark.parametrize("is_rms", [False, True])
def test_fwd_bwd(hk, cuda, combo, shape, features, is_rms):
    import torch
    wt, it, rt = combo
    if features == "types-only" and wt == it == rt:
        pytest.skip("uniform types without features take the plain kernels (tested elsewhere)")
    rows, cols = shape
    eps = 1e-5
    seed = 7000 + cols + rows
    p = 0.2 if features in ("dropout", "all") else 0.0
    x0 = helpers.draw(seed, (rows, cols), dtype=it)
    residual = helpers.draw(seed + 1, (rows, cols), dtype=rt) if features in ("all", "types-only") else None
    gamma = helpers.draw(seed + 2, (cols,), "uniform", 0.5, 1.5, wt)
    beta = None if is_rms else helpers.draw(seed + 3, (cols,), "normal", 0.0, 0.1, wt)
    rowscale = helpers.draw(seed + 4, (rows,), "uniform", 0.5, 2.0, it) if features in ("scales", "all") else None
    colscale = helpers.draw(seed + 5, (cols,), "uniform", 0.5, 2.0, wt) if features in ("scales", "all") else None
    dz = helpers.draw(seed + 6, (rows, cols), dtype=it)
    dx_in = helpers.draw(seed + 7, (rows, cols), dtype=rt) if features == "all" else None
    emask = _mask(rows * cols, p).reshape(rows, cols) if p > 0 else None

    ez, ex, emu, ers = dal.fwd(x0, residual, gamma, beta, rowscale, colscale, dmask=emask, dropout_p=p, eps=eps,
                               is_rms=is_rms)
    tx0, tg, tb = _tt(x0, it, cuda), _tt(gamma, wt, cuda), _tt(beta, wt, cuda)
    tres, trow, tcol = _tt(residual, rt, cuda), _tt(rowscale, it, cuda), _tt(colscale, wt, cuda)
    tz = torch.empty_like(tx0)
    tx = torch.empty(rows, cols, dtype=helpers.to_torch(np.zeros(1, np.float32), rt, "cpu").dtype, device=cuda)
    tmu = torch.empty(rows, dtype=torch.float32, device=cuda)
    trs = torch.empty(rows, dtype=torch.float32, device=cuda)
    tmask = torch.full((rows, cols), 7, dtype=torch.uint8, device=cuda) if p > 0 else None
    hk.dropout_add_ln_fwd_ex(tx0, tg, tz, tmu, trs, residual=tres, beta=tb, rowscale=trow, colscale=tcol, x=tx,
                             dmask=tmask, dropout_p=p, eps=eps, is_rms=is_rms, seed=SEED, offset=OFFSET)
    torch.cuda.synchronize()
    if p > 0:
        assert np.array_equal(tmask.cpu().numpy(), emask), "keep mask differs from the oracle's"
    helpers.assert_close(tz, ez, it, "z")
    helpers.assert_close(tx, ex, rt, "x")
    helpers.assert_close(tmu, emu, "fp32", "mu", scale=float(np.sqrt(np.mean(ex ** 2))))
    helpers.assert_close(trs, ers, "fp32", "rs")

    # backward from the statistics and the pre-norm sum as a forward stores them
    xs = oracle.round_to(ex.astype(np.float32), rt)
    mu32, rs32 = emu.astype(np.float32), ers.astype(np.float32)
    edx0, edres, edg, edb, edcol = dal.bwd(dz, dx_in, xs, x0, emask, mu32, rs32, gamma, rowscale, colscale,
                                           dropout_p=p, is_rms=is_rms)
    tdz, tdxin, txs = _tt(dz, it, cuda), _tt(dx_in, rt, cuda), _tt(xs, rt, cuda)
    tdx0 = torch.empty_like(tx0)
    tdres = torch.empty_like(txs)
    tdg, tdb = torch.empty_like(tg), torch.empty_like(tg)
    tdcol = torch.empty_like(tg) if colscale is not None else None
    hk.dropout_add_ln_bwd_ex(tdz, txs, _tt(mu32, "fp32", cuda), _tt(rs32, "fp32", cuda), tg, tdx0, dx=tdxin,
                             x0=tx0, dmask=_tt(emask, "uint8", cuda), rowscale=trow, colscale=tcol,
                             dresidual=tdres, dgamma=tdg, dbeta=tdb, dcolscale=tdcol, dropout_p=p, is_rms=is_rms)
    torch.cuda.synchronize()
    helpers.assert_close(tdx0, edx0, it, "dx0")
    helpers.assert_close(tdres, edres, rt, "dresidual")
    helpers.assert_close(tdg, edg, wt, "dgamma")
    helpers.assert_close(tdb, edb, wt, "dbeta")
    if colscale is not None:
        helpers.assert_close(tdcol, edcol, wt, "dcolscale")
    if p > 0:
        assert (helpers.to_numpy(tdx0)[emask == 0] == 0).all(), "dropped elements must get a zero gradient"


@pytest.mark.parametrize("combo", [("fp32", "fp32", "fp32"), ("bf16", "bf16", "bf16"), ("fp32", "bf16", "fp32")],
                         ids=lambda c: "w%s-i%s-r%s" % c)
@pytest.mark.parametrize("p", [0.0, 0.3])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("cols", [256, 4096])
def test_row_subsets(hk, cuda, combo, p, is_rms, cols):
    import torch
    wt, it, rt = combo
    rows, x0_rows, z_rows, eps, rsc = 37, 23, 19, 1e-5, 0.75
    g = helpers.rng(99 + cols)
    # every x0 row and every z row is referenced exactly once, the other rows of the sum have none;
    # two entries are out of range and must be treated as "no row"
    x0_subset = np.zeros(rows, dtype=np.int32)
    x0_subset[g.permutation(rows)[:x0_rows]] = np.arange(1, x0_rows + 1)
    z_subset = np.zeros(rows, dtype=np.int32)
    z_subset[g.permutation(rows)[:z_rows]] = np.arange(1, z_rows + 1)
    free_x0 = np.flatnonzero(x0_subset == 0)
    x0_bad = x0_subset.copy(); x0_bad[free_x0[0]] = x0_rows + 5; x0_bad[free_x0[1]] = -3
    free_z = np.flatnonzero(z_subset == 0)
    z_bad = z_subset.copy(); z_bad[free_z[0]] = z_rows + 1

    x0 = helpers.draw(1, (x0_rows, cols), dtype=it)
    residual = helpers.draw(2, (rows, cols), dtype=rt)
    gamma = helpers.draw(3, (cols,), "uniform", 0.5, 1.5, wt)
    beta = helpers.draw(4, (cols,), "normal", 0.0, 0.1, wt)
    colscale = helpers.draw(5, (cols,), "uniform", 0.5, 2.0, wt)
    rowscale_ignored = helpers.draw(6, (rows,), "uniform", 5.0, 6.0, it)   # subsets use rowscale_const
    dz = helpers.draw(7, (z_rows, cols), dtype=it)
    dx_in = helpers.draw(8, (rows, cols), dtype=rt)
    emask = _mask(x0_rows * cols, p).reshape(x0_rows, cols) if p > 0 else None

    ez, ex, emu, ers = dal.fwd(x0, residual, gamma, beta, None, colscale, x0_subset, z_subset, emask, p, eps, rsc,
                               z_rows, is_rms)
    tdt = lambda name: helpers.to_torch(np.zeros(1, np.float32), name, "cpu").dtype
    tx0, tres, tg, tb, tcol = (_tt(v, d, cuda) for v, d in ((x0, it), (residual, rt), (gamma, wt), (beta, wt),
                                                            (colscale, wt)))
    tz = torch.zeros(z_rows, cols, dtype=tdt(it), device=cuda)
    tx = torch.empty(rows, cols, dtype=tdt(rt), device=cuda)
    tmu = torch.empty(rows, dtype=torch.float32, device=cuda); trs = torch.empty_like(tmu)
    tmask = torch.zeros(x0_rows, cols, dtype=torch.uint8, device=cuda) if p > 0 else None
    sx0, sz = _tt(x0_bad, "int32", cuda), _tt(z_bad, "int32", cuda)
    hk.dropout_add_ln_fwd_ex(tx0, tg, tz, tmu, trs, residual=tres, beta=tb, colscale=tcol, x=tx, dmask=tmask,
                             rowscale=_tt(rowscale_ignored, it, cuda), x0_subset=sx0, z_subset=sz, dropout_p=p,
                             eps=eps, rowscale_const=rsc, is_rms=is_rms, seed=SEED, offset=OFFSET)
    torch.cuda.synchronize()
    if p > 0:
        assert np.array_equal(tmask.cpu().numpy(), emask)
    helpers.assert_close(tz, ez, it, "z")        # every z row is written (no NaN left in the oracle's z)
    helpers.assert_close(tx, ex, rt, "x")
    helpers.assert_close(trs, ers, "fp32", "rs")

    xs = oracle.round_to(ex.astype(np.float32), rt)
    mu32, rs32 = emu.astype(np.float32), ers.astype(np.float32)
    edx0, edres, edg, edb, edcol = dal.bwd(dz, dx_in, xs, x0, emask, mu32, rs32, gamma, None, colscale, x0_subset,
                                           z_subset, p, rsc, x0_rows, is_rms)
    tdx0 = torch.zeros(x0_rows, cols, dtype=tdt(it), device=cuda)
    tdres = torch.empty(rows, cols, dtype=tdt(rt), device=cuda)
    tdg, tdb, tdcol = torch.empty_like(tg), torch.empty_like(tg), torch.empty_like(tg)
    hk.dropout_add_ln_bwd_ex(_tt(dz, it, cuda), _tt(xs, rt, cuda), _tt(mu32, "fp32", cuda),
                             _tt(rs32, "fp32", cuda), tg, tdx0, dx=_tt(dx_in, rt, cuda), x0=tx0,
                             dmask=_tt(emask, "uint8", cuda), colscale=tcol, x0_subset=sx0, z_subset=sz,
                             dresidual=tdres, dgamma=tdg, dbeta=tdb, dcolscale=tdcol, dropout_p=p,
                             rowscale_const=rsc, is_rms=is_rms)
    torch.cuda.synchronize()
    helpers.assert_close(tdx0, edx0, it, "dx0")
    helpers.assert_close(tdres, edres, rt, "dresidual")
    helpers.assert_close(tdg, edg, wt, "dgamma")
    helpers.assert_close(tdb, edb, wt, "dbeta")
    helpers.assert_close(tdcol, edcol, wt, "dcolscale")


@pytest.mark.parametrize("combo", [("fp32", "fp32", "fp32"), ("fp16", "fp16", "fp16"), ("bf16", "bf16", "fp32"),
                                   ("fp32", "bf16", "bf16")], ids=lambda c: "w%s-i%s-r%s" % c)
@pytest.mark.parametrize("has_x1,tied", [(True, False), (True, True), (False, False)])
@pytest.mark.parametrize("p", [0.0, 0.25])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("shape", [(21, 512), (7, 5120)], ids=lambda s: "%dx%d" % s)
def test_parallel_residual(hk, cuda, combo, has_x1, tied, p, is_rms, shape):
    import torch
    wt, it, rt = combo
    rows, cols = shape
    eps = 1e-5
    x0 = helpers.draw(11, (rows, cols), dtype=it)
    x1 = helpers.draw(12, (rows, cols), dtype=it) if has_x1 else None
    residual = helpers.draw(13, (rows, cols), dtype=rt)
    g0 = helpers.draw(14, (cols,), "uniform", 0.5, 1.5, wt); b0 = helpers.draw(15, (cols,), "normal", 0.0, 0.1, wt)
    g1 = None if tied else helpers.draw(16, (cols,), "uniform", 0.5, 1.5, wt)
    b1 = None if tied else helpers.draw(17, (cols,), "normal", 0.0, 0.1, wt)
    dz0 = helpers.draw(18, (rows, cols), dtype=it)
    dz1 = None if tied else helpers.draw(19, (rows, cols), dtype=it)
    dx_in = helpers.draw(20, (rows, cols), dtype=rt)
    m0 = _mask(rows * cols, p, 0).reshape(rows, cols) if p > 0 else None
    m1 = _mask(rows * cols, p, 1).reshape(rows, cols) if p > 0 and has_x1 else None

    ez0, ez1, ex, emu, ers = dal.parallel_fwd(x0, x1, residual, g0, b0, g1, b1, m0, m1, p, eps, is_rms)
    tdt = lambda name: helpers.to_torch(np.zeros(1, np.float32), name, "cpu").dtype
    tx0, tx1, tres = _tt(x0, it, cuda), _tt(x1, it, cuda), _tt(residual, rt, cuda)
    tg0, tb0, tg1, tb1 = _tt(g0, wt, cuda), _tt(b0, wt, cuda), _tt(g1, wt, cuda), _tt(b1, wt, cuda)
    tz0 = torch.empty_like(tx0); tz1 = None if tied else torch.empty_like(tx0)
    tx = torch.empty(rows, cols, dtype=tdt(rt), device=cuda)
    tmu = torch.empty(rows, dtype=torch.float32, device=cuda); trs = torch.empty_like(tmu)
    tm0 = torch.zeros(rows, cols, dtype=torch.uint8, device=cuda) if p > 0 else None
    tm1 = torch.zeros(rows, cols, dtype=torch.uint8, device=cuda) if p > 0 and has_x1 else None
    hk.dropout_add_ln_fwd_ex(tx0, tg0, tz0, tmu, trs, x1=tx1, residual=tres, beta=tb0, gamma1=tg1, beta1=tb1,
                             z1=tz1, x=tx, dmask=tm0, dmask1=tm1, dropout_p=p, eps=eps, is_rms=is_rms, seed=SEED,
                             offset=OFFSET)
    torch.cuda.synchronize()
    if p > 0:
        assert np.array_equal(tm0.cpu().numpy(), m0)
        if has_x1:
            assert np.array_equal(tm1.cpu().numpy(), m1)
            assert 0.2 < (m0 != m1).mean() < 0.5   # independent streams: differ with probability 2 p (1 - p)
    helpers.assert_close(tz0, ez0, it, "z0")
    if not tied:
        helpers.assert_close(tz1, ez1, it, "z1")
    helpers.assert_close(tx, ex, rt, "x")
    helpers.assert_close(trs, ers, "fp32", "rs")

    xs = oracle.round_to(ex.astype(np.float32), rt)
    mu32, rs32 = emu.astype(np.float32), ers.astype(np.float32)
    edx0, edx1, edres, edg0, edb0, edg1, edb1 = dal.parallel_bwd(dz0, dz1, dx_in, xs, m0, m1, mu32, rs32, g0, g1, p,
                                                                 has_x1, is_rms)
    tdx0 = torch.empty_like(tx0); tdx1 = torch.empty_like(tx0) if has_x1 else None
    tdres = torch.empty(rows, cols, dtype=tdt(rt), device=cuda)
    tdg0, tdb0 = torch.empty_like(tg0), torch.empty_like(tg0)
    tdg1 = None if tied else torch.empty_like(tg0); tdb1 = None if tied else torch.empty_like(tg0)
    hk.dropout_add_ln_bwd_ex(_tt(dz0, it, cuda), _tt(xs, rt, cuda), _tt(mu32, "fp32", cuda),
                             _tt(rs32, "fp32", cuda), tg0, tdx0, dz1=_tt(dz1, it, cuda), dx=_tt(dx_in, rt, cuda),
                             dmask=_tt(m0, "uint8", cuda), dmask1=_tt(m1, "uint8", cuda), gamma1=tg1, dx1=tdx1,
                             dresidual=tdres, dgamma=tdg0, dbeta=tdb0, dgamma1=tdg1, dbeta1=tdb1, dropout_p=p,
                             is_rms=is_rms)
    torch.cuda.synchronize()
    helpers.assert_close(tdx0, edx0, it, "dx0")
    if has_x1:
        helpers.assert_close(tdx1, edx1, it, "dx1")
    helpers.assert_close(tdres, edres, rt, "dresidual")
    helpers.assert_close(tdg0, edg0, wt, "dgamma0")
    helpers.assert_close(tdb0, edb0, wt, "dbeta0")
    if not tied:
        helpers.assert_close(tdg1, edg1, wt, "dgamma1")
        helpers.assert_close(tdb1, edb1, wt, "dbeta1")


@pytest.mark.parametrize("combo", COMBOS, ids=lambda c: "w%s-i%s-r%s" % c)
@pytest.mark.parametrize("rows,cols,blocks", [(1, 512, 0), (61, 512, 2), (50, 4096, 3), (2500, 4096, 0),
                                               (37, 5120, 5), (19, 8192, 4), (23, 1000, 2)])
@pytest.mark.parametrize("is_rms", [False, True])
def test_prenorm_block_backward(hk, cuda, combo, rows, cols, blocks, is_rms):
    """Dropout + incoming and outgoing residual-stream gradients and nothing else: the form with a kernel of
    its own when the row fills every thread (cols = 1000 does not and takes the general kernel).  A forced
    small grid makes every thread group walk many rows, through full rounds and the guarded tail."""
    import torch
    wt, it, rt = combo
    p = 0.15
    seed = 8100 + rows + cols
    x = helpers.draw(seed, (rows, cols), dtype=rt)
    gamma = helpers.draw(seed + 1, (cols,), "uniform", 0.5, 1.5, wt)
    dz = helpers.draw(seed + 2, (rows, cols), dtype=it)
    dx_in = helpers.draw(seed + 3, (rows, cols), dtype=rt)
    mask = _mask(rows * cols, p).reshape(rows, cols)
    xd = x.astype(np.float64)
    mu = xd.mean(axis=1)
    rs = 1.0 / np.sqrt((xd * xd).mean(axis=1) + 1e-5) if is_rms else 1.0 / np.sqrt(xd.var(axis=1) + 1e-5)
    mu32, rs32 = mu.astype(np.float32), rs.astype(np.float32)
    edx0, edres, edg, edb, _ = dal.bwd(dz, dx_in, x, None, mask, mu32, rs32, gamma, dropout_p=p, is_rms=is_rms)
    tx, tdxin = _tt(x, rt, cuda), _tt(dx_in, rt, cuda)
    tdz, tg = _tt(dz, it, cuda), _tt(gamma, wt, cuda)
    tdx0 = torch.empty_like(tdz); tdres = torch.empty_like(tx)
    tdg, tdb = torch.empty_like(tg), torch.empty_like(tg)
    hk.tune_set("norm_bwd_blocks", blocks)
    try:
        hk.dropout_add_ln_bwd_ex(tdz, tx, _tt(mu32, "fp32", cuda), _tt(rs32, "fp32", cuda), tg, tdx0, dx=tdxin,
                                 dmask=_tt(mask, "uint8", cuda), dresidual=tdres, dgamma=tdg, dbeta=tdb,
                                 dropout_p=p, is_rms=is_rms)
        torch.cuda.synchronize()
    finally:
        hk.tune_set("norm_bwd_blocks", 0)
    helpers.assert_close(tdx0, edx0, it, "dx0")
    helpers.assert_close(tdres, edres, rt, "dresidual")
    helpers.assert_close(tdg, edg, wt, "dgamma")
    helpers.assert_close(tdb, edb, wt, "dbeta")
    assert (helpers.to_numpy(tdx0)[mask == 0] == 0).all()


def test_plain_call_matches_the_plain_entry_point(hk, cuda):
    """No feature and uniform types: the call is handed to the tuned kernels, bit for bit."""
    import torch
    rows, cols = 64, 4096
    x = helpers.to_torch(helpers.draw(1, (rows, cols), dtype="bf16"), "bf16", cuda)
    g = helpers.to_torch(helpers.draw(2, (cols,), "uniform", 0.5, 1.5, "bf16"), "bf16", cuda)
    dz = helpers.to_torch(helpers.draw(3, (rows, cols), dtype="bf16"), "bf16", cuda)
    out = []
    for fn in ("plain", "ex"):
        z = torch.empty_like(x); mu = torch.empty(rows, dtype=torch.float32, device=cuda); rs = torch.empty_like(mu)
        dx = torch.empty_like(x); dg = torch.empty_like(g); db = torch.empty_like(g)
        if fn == "plain":
            hk.dropout_add_ln_fwd(x, None, g, None, z, None, mu, rs, 1e-6, True)
            hk.dropout_add_ln_bwd(dz, None, x, mu, rs, g, dx, None, dg, db, True)
        else:
            hk.dropout_add_ln_fwd_ex(x, g, z, mu, rs, eps=1e-6, is_rms=True)
            hk.dropout_add_ln_bwd_ex(dz, x, mu, rs, g, dx, dgamma=dg, dbeta=db, is_rms=True)
        torch.cuda.synchronize()
        out.append((z, mu, rs, dx, dg, db))
    for a, b in zip(*out):
        assert torch.equal(a, b)


def test_mask_at_scale(hk, cuda):
    """2048 x 4096 elements: the mask equals the oracle's bit for bit, is reproducible, depends on seed and
    offset, keeps a fraction within 5 sigma of 1 - p, and a dropped element reaches neither x nor dx0."""
    import torch
    rows, cols, p = 2048, 4096, 0.1
    x0 = torch.randn(rows, cols, device=cuda, dtype=torch.bfloat16)
    g = torch.ones(cols, device=cuda, dtype=torch.bfloat16)
    z = torch.empty_like(x0); x = torch.empty_like(x0)
    mu = torch.empty(rows, dtype=torch.float32, device=cuda); rs = torch.empty_like(mu)

    def run(seed, offset):
        m = torch.zeros(rows, cols, dtype=torch.uint8, device=cuda)
        hk.dropout_add_ln_fwd_ex(x0, g, z, mu, rs, x=x, dmask=m, dropout_p=p, is_rms=True, seed=seed, offset=offset)
        torch.cuda.synchronize()
        return m

    m = run(SEED, OFFSET)
    assert np.array_equal(m.cpu().numpy().reshape(-1), _mask(rows * cols, p))
    assert torch.equal(m, run(SEED, OFFSET))
    n = rows * cols
    assert abs(m.float().mean().item() - (1 - p)) < 5 * np.sqrt(p * (1 - p) / n)
    kept = x0.float() * (1.0 / (1.0 - p))
    assert torch.equal(x[m == 0], torch.zeros_like(x[m == 0]))
    assert torch.allclose(x[m == 1].float(), kept[m == 1], rtol=1e-2)
    for other in (run(SEED + 1, OFFSET), run(SEED, OFFSET + 1)):
        frac = (other != m).float().mean().item()
        assert abs(frac - 2 * p * (1 - p)) < 0.01


def test_refused_calls(hk, cuda):
    import torch
    x = torch.zeros(4, 256, device=cuda, dtype=torch.bfloat16)
    g = torch.ones(256, device=cuda, dtype=torch.bfloat16)
    z = torch.empty_like(x); mu = torch.empty(4, dtype=torch.float32, device=cuda); rs = torch.empty_like(mu)
    m = torch.zeros(4, 256, dtype=torch.uint8, device=cuda)
    sub = torch.ones(4, dtype=torch.int32, device=cuda)
    with pytest.raises(hk.HkError) as e:       # dropout without a mask buffer
        hk.dropout_add_ln_fwd_ex(x, g, z, mu, rs, dropout_p=0.1)
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # p outside [0, 1)
        hk.dropout_add_ln_fwd_ex(x, g, z, mu, rs, dmask=m, dropout_p=1.0)
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # one subset without the other
        hk.dropout_add_ln_fwd_ex(x, g, z, mu, rs, x0_subset=sub)
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # the parallel form has no column scaling
        hk.dropout_add_ln_fwd_ex(x, g, z, mu, rs, x1=x, colscale=g)
    assert e.value.code == -2
    with pytest.raises(hk.HkError) as e:       # bf16 weights with fp32 input: not a registered combination
        hk.dropout_add_ln_fwd_ex(x.float(), g, z.float(), mu, rs, colscale=g)
    assert e.value.code == -2
    with pytest.raises(hk.HkError) as e:       # hidden size not a multiple of 8
        hk.dropout_add_ln_fwd_ex(x[:, :252].contiguous(), g[:252].contiguous(), z[:, :252].contiguous(), mu, rs,
                                 dmask=m, dropout_p=0.1)
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # hidden size above 8192
        big = torch.zeros(2, 8200, device=cuda, dtype=torch.bfloat16)
        hk.dropout_add_ln_fwd_ex(big, torch.ones(8200, device=cuda, dtype=torch.bfloat16), torch.empty_like(big),
                                 mu[:2], rs[:2], colscale=torch.ones(8200, device=cuda, dtype=torch.bfloat16))
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # column scaling in the backward needs x0
        hk.dropout_add_ln_bwd_ex(x, x, mu, rs, g, z, colscale=g, dcolscale=torch.empty_like(g))
    assert e.value.code == -1
    with pytest.raises(hk.HkError) as e:       # workspace too small
        hk.dropout_add_ln_bwd_ex(x, x, mu, rs, g, z, dmask=m, dropout_p=0.1, dgamma=torch.empty_like(g),
                                 workspace=torch.empty(4, device=cuda))
    assert e.value.code == -4
    # zero rows: nothing to do in the forward, zero column sums in the backward
    e0 = x[:0]
    hk.dropout_add_ln_fwd_ex(e0, g, e0.clone(), mu[:0], rs[:0], dmask=m[:0], dropout_p=0.1)
    dg = torch.full_like(g, 3.0)
    hk.dropout_add_ln_bwd_ex(e0, e0, mu[:0], rs[:0], g, e0.clone(), dmask=m[:0], dropout_p=0.1, dgamma=dg)
    torch.cuda.synchronize()
    assert (dg == 0).all()
