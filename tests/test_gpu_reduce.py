"""GPU parity of Reduce sum / mean over arbitrary axes (hk_reduce)."""
import itertools

import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu


def _run(hk, cuda, tx, axes, op, out_dtype=None):
    import torch
    red = sorted(set(axes))
    out_shape = [s for d, s in enumerate(tx.shape) if d not in red] or [1]
    out = torch.full(out_shape, -7, dtype=out_dtype or tx.dtype, device=cuda)
    hk.reduce(tx, out, list(axes), op)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_every_axis_subset_is_exact(hk, cuda, dtype):
    """Small integers make every fp32 partial sum exact: results are known bit for bit,
    whatever order the kernels add in.  Covers the dimension-merging rule."""
    shape = (3, 4, 5, 6)
    x = helpers.rng(7).integers(-3, 4, size=shape).astype(np.float32)
    tx = helpers.to_torch(x, dtype, cuda)
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            want = x.astype(np.float64).sum(axis=axes)
            got = _run(hk, cuda, tx, axes, "sum")
            assert np.array_equal(helpers.to_numpy(got).astype(np.float64).reshape(want.shape or (1,)),
                                  want.reshape(want.shape or (1,))), axes
    # unsorted and repeated axes are sorted and de-duplicated
    got = _run(hk, cuda, tx, [2, 0, 2], "sum")
    assert np.array_equal(helpers.to_numpy(got), x.sum(axis=(0, 2)))


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("shape,axes", [((512, 4096), (0,)), ((512, 4096), (1,)), ((8, 64, 4096), (0, 1)),
                                        ((6, 300, 520), (1,)), ((5, 1000), (1,)), ((1000, 5), (0,)),
                                        ((3, 100000), (1,)), ((70000,), (0,)), ((4, 33, 7), (0, 2)),
                                        ((33, 264), (0,)), ((2, 2, 1 << 20), (2,))])
@pytest.mark.parametrize("op", ["sum", "mean"])
def test_reduce_parity(hk, cuda, dtype, shape, axes, op):
    x = helpers.draw(301, shape, dtype=dtype)
    want = oracle.reduce(x, list(axes), op)
    tx = helpers.to_torch(x, dtype, cuda)
    got = _run(hk, cuda, tx, axes, op)
    n = int(np.prod([shape[a] for a in axes]))
    helpers.assert_close(got, want, dtype, "%s %s" % (op, axes), scale=float(np.sqrt(n)) / (n if op == "mean" else 1))


def test_mean_rounding_order(hk, cuda):
    """mean = fp32 sum * float(1/n): integer inputs make the sum exact, so the result is known bit for bit."""
    x = helpers.rng(11).integers(-8, 9, size=(64, 3000)).astype(np.float32)
    tx = helpers.to_torch(x, "fp32", cuda)
    got = helpers.to_numpy(_run(hk, cuda, tx, (1,), "mean"))
    want = oracle.reduce(x, [1], "mean", mean_mode=1).astype(np.float32)
    assert np.array_equal(got, want)


def test_strided_views_and_fp32_output(hk, cuda):
    import torch
    x = helpers.draw(302, (16, 24, 40), dtype="bf16")
    tx = helpers.to_torch(x, "bf16", cuda)
    for view, nview in ((tx.permute(2, 0, 1), x.transpose(2, 0, 1)), (tx[:, ::2, 3:35], x[:, ::2, 3:35]),
                        (tx.transpose(0, 1), x.transpose(1, 0, 2))):
        for axes in ((0,), (1,), (2,), (0, 2), (0, 1, 2)):
            want = oracle.reduce(np.ascontiguousarray(nview), list(axes), "sum")
            got = _run(hk, cuda, view, axes, "sum", out_dtype=torch.float32)
            helpers.assert_close(got, want, "fp32", "strided %s" % (axes,), scale=float(np.abs(want).max()), rtol=1e-5)


@pytest.mark.parametrize("tdt", ["int64", "int32", "fp64", "uint8"])
def test_integer_and_double(hk, cuda, tdt):
    import torch
    x = helpers.rng(5).integers(0, 5, size=(17, 33, 9))
    tx = torch.from_numpy(x).to(hk.torch_dtype(tdt)).to(cuda)
    for axes in ((0,), (1, 2), (0, 1, 2), (2,)):
        got = _run(hk, cuda, tx, axes, "sum")
        want = x.sum(axis=axes)
        if tdt == "uint8":
            want = want % 256
        assert np.array_equal(got.cpu().numpy().astype(np.int64).reshape(-1), np.asarray(want).reshape(-1))


def test_full_size_configs(hk, cuda):
    import torch
    g = torch.Generator(device="cpu").manual_seed(301)
    tx = torch.randn((32768, 4096), generator=g, dtype=torch.float32).to(torch.bfloat16).to(cuda)
    xd = tx.double()
    for axes, op in (((0,), "sum"), ((0,), "mean"), ((1,), "sum"), ((1,), "mean")):
        want = (xd.sum(axes[0]) if op == "sum" else xd.mean(axes[0])).cpu().numpy()
        got = _run(hk, cuda, tx, axes, op)
        n = tx.shape[axes[0]]
        helpers.assert_close(got, want, "bf16", "%s %s" % (op, axes), scale=float(np.sqrt(n)) / (n if op == "mean" else 1))
    t3 = tx.view(64, 512, 4096)
    got = _run(hk, cuda, t3, (0, 1), "sum")
    helpers.assert_close(got, xd.sum(0).cpu().numpy(), "bf16", "sum (0,1)", scale=float(np.sqrt(32768)))
    # linearity: sum(2x) == 2 sum(x) exactly in bf16 (scaling by two is exact)
    got2 = _run(hk, cuda, (tx * 2), (0,), "sum")
    assert torch.equal(got2.float(), _run(hk, cuda, tx, (0,), "sum").float() * 2)


def test_degenerate_reductions(hk, cuda):
    """No axes = a dense copy (also of a strided view); a reduced extent of 0 gives
    the empty sum 0 and the empty mean NaN; nothing kept = nothing written."""
    import torch
    x = helpers.draw(11, (6, 10), dtype="fp32")
    tx = helpers.to_torch(x, "fp32", cuda)
    got = _run(hk, cuda, tx, (), "sum")
    assert np.array_equal(helpers.to_numpy(got), x)
    view = tx.t()
    out = torch.full((10, 6), -7.0, device=cuda)
    hk.reduce(view, out, [], "sum")
    torch.cuda.synchronize()
    assert np.array_equal(helpers.to_numpy(out), x.T)
    empty = torch.empty((0, 10), device=cuda)
    assert np.array_equal(helpers.to_numpy(_run(hk, cuda, empty, (0,), "sum")), np.zeros(10, dtype=np.float32))
    assert np.all(np.isnan(helpers.to_numpy(_run(hk, cuda, empty, (0,), "mean"))))
    assert np.all(np.isnan(helpers.to_numpy(_run(hk, cuda, empty.bfloat16(), (0,), "mean"))))
    untouched = torch.full((1,), -7.0, device=cuda)
    hk.reduce(torch.empty((10, 0), device=cuda), torch.empty((0,), device=cuda), [0], "sum")
    torch.cuda.synchronize()
    assert float(untouched[0]) == -7.0


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("op", ["max", "min"])
def test_max_min_are_exact_selections(hk, cuda, dtype, op):
    """A maximum / minimum is one of the inputs: the result is known bit for bit in every dtype, whatever
    order the kernels combine in.  Covers the row, column, split and generic kernels."""
    import itertools
    shape = (3, 4, 5, 6)
    x = helpers.draw(21, shape, dtype=dtype)
    tx = helpers.to_torch(x, dtype, cuda)
    f = np.max if op == "max" else np.min
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            got = helpers.to_numpy(_run(hk, cuda, tx, axes, op)).astype(np.float64)
            assert np.array_equal(got.reshape(-1), np.asarray(f(x.astype(np.float64), axis=axes)).reshape(-1)), axes
    for shp, axes in (((257, 4096), (0,)), ((257, 4096), (1,)), ((3, 70000), (1,)), ((20000, 72), (0,)),
                      ((64, 33, 40), (0, 2)), ((5, 1000, 24), (1,)), ((1, 16384), (1,)), ((9, 1031), (1,))):
        x = helpers.draw(22 + len(shp), shp, dtype=dtype)
        tx = helpers.to_torch(x, dtype, cuda)
        got = helpers.to_numpy(_run(hk, cuda, tx, axes, op)).astype(np.float64)
        assert np.array_equal(got.reshape(-1), np.asarray(f(x.astype(np.float64), axis=axes)).reshape(-1)), (shp, axes)
    # a strided view
    base = helpers.to_torch(helpers.draw(29, (48, 20, 64), dtype=dtype), dtype, cuda)
    view = base.permute(1, 2, 0)[:, ::2, :]
    want = f(helpers.to_numpy(view.contiguous()).astype(np.float64), axis=(0, 2))
    assert np.array_equal(helpers.to_numpy(_run(hk, cuda, view, (0, 2), op)).astype(np.float64).reshape(-1), want.reshape(-1))


@pytest.mark.parametrize("op", ["max", "min"])
def test_max_min_nan_and_infinities(hk, cuda, op):
    import torch
    x = helpers.draw(31, (64, 4096), dtype="fp32")
    x[3, 100] = np.nan
    x[5, 7] = np.inf
    x[6, 9] = -np.inf
    tx = helpers.to_torch(x, "fp32", cuda)
    for axes in ((1,), (0,)):
        got = helpers.to_numpy(_run(hk, cuda, tx, axes, op)).astype(np.float64).reshape(-1)
        want = np.asarray(oracle.reduce(x, list(axes), op)).reshape(-1)
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(want).sum() == 1
        assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    # an empty reduced extent writes the identity
    empty = torch.empty((0, 10), device=cuda)
    ident = -np.inf if op == "max" else np.inf
    assert np.all(helpers.to_numpy(_run(hk, cuda, empty, (0,), op)) == ident)
    assert np.all(helpers.to_numpy(_run(hk, cuda, empty.bfloat16(), (0,), op)).astype(np.float64) == ident)
    # integers: exact, identities are the type's extremes
    xi = helpers.rng(32).integers(-1000, 1000, size=(17, 33, 9))
    for tdt in ("int64", "int32", "uint8"):
        ti = torch.from_numpy(xi).to(hk.torch_dtype(tdt)).to(cuda)
        ref = ti.cpu().numpy()
        got = _run(hk, cuda, ti, (0, 2), op).cpu().numpy()
        assert np.array_equal(got, (ref.max(axis=(0, 2)) if op == "max" else ref.min(axis=(0, 2)))), tdt


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_prod_parity_and_widened_output(hk, cuda, dtype):
    import torch
    # factors near 1 keep long products in range; fp32 accumulation against the float64 oracle
    for shp, axes in (((300, 512), (1,)), ((300, 512), (0,)), ((7, 40, 24), (0, 2)), ((2, 3), (0, 1))):
        x = helpers.draw(41 + len(shp), shp, "uniform", 0.97, 1.03, dtype)
        tx = helpers.to_torch(x, dtype, cuda)
        want = np.asarray(oracle.reduce(x, list(axes), "prod"))
        helpers.assert_close(_run(hk, cuda, tx, axes, "prod"), want, dtype, "prod %s %s" % (shp, axes))
        if dtype == "bf16":
            helpers.assert_close(_run(hk, cuda, tx, axes, "prod", out_dtype=torch.float32), want, "fp32",
                                 "prod to fp32 %s %s" % (shp, axes), rtol=2e-5)
    # small integers: exact
    xi = helpers.rng(43).integers(1, 4, size=(6, 5)).astype(np.float32)
    got = helpers.to_numpy(_run(hk, cuda, helpers.to_torch(xi, "fp32", cuda), (1,), "prod"))
    assert np.array_equal(got, xi.prod(axis=1))
    assert np.all(helpers.to_numpy(_run(hk, cuda, torch.empty((4, 0), device=cuda), (1,), "prod")) == 1.0)
    # max / min have no widened output
    with pytest.raises(hk.HkError):
        _run(hk, cuda, helpers.to_torch(xi, "bf16", cuda), (1,), "max", out_dtype=torch.float32)


def test_split_column_reduction_on_many_streams(hk, cuda):
    """A column reduction whose rows are split over workgroups gives the same bits eagerly and as a graph replay, on
    every one of 40 streams whose calls overlap, call after call, with calls of other shapes in between."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(77)
    shapes = [(4096, 4096), (2048, 512), (3000, 1032), (4, 1024, 2048)]
    xs = [torch.randn(*s, generator=g, device=cuda).to(torch.bfloat16) for s in shapes]
    axes = [[0], [0], [0], [1]]
    # reference: a graph replay
    want = []
    for x, ax in zip(xs, axes):
        kept = [d for i, d in enumerate(x.shape) if i not in ax]
        out = torch.empty(kept, dtype=torch.bfloat16, device=cuda)
        ws = torch.empty(max(1, hk.reduce_workspace_bytes(8, list(x.shape), list(x.stride()), ax) // 4 + 4), device=cuda)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            hk.reduce(x, out, ax, "sum", workspace=ws)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            hk.reduce(x, out, ax, "sum", workspace=ws)
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want.append(out.clone())
        # against float64 sums as well
        ref = x.double().sum(dim=ax[0])
        assert float(((out.double() - ref).abs() / (ref.abs() + ref.abs().mean())).max()) < 1e-2
    streams = [torch.cuda.Stream() for _ in range(40)]
    outs = [[torch.empty_like(w) for w in want] for _ in streams]
    wss = [[torch.empty(max(1, hk.reduce_workspace_bytes(8, list(x.shape), list(x.stride()), ax) // 4 + 4), device=cuda)
            for x, ax in zip(xs, axes)] for _ in streams]
    for rep in range(3):
        for si, st in enumerate(streams):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                for k, (x, ax) in enumerate(zip(xs, axes)):
                    outs[si][k].fill_(float("nan"))
                    hk.reduce(x, outs[si][k], ax, "sum", workspace=wss[si][k])
        torch.cuda.synchronize()
        for si in range(len(streams)):
            for k in range(len(xs)):
                assert torch.equal(outs[si][k].view(torch.int16), want[k].view(torch.int16)), (rep, si, k)
