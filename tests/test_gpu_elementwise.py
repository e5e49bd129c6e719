"""GPU parity of the element-wise operators (hk_unary, hk_binary_const, hk_binary) and of the
vocabulary-parallel cross-entropy's local kernels (hk_vocab_parallel_ce_gather / _bwd) through the C-ABI.
The expected values are numpy float64 one-liners of the operator's definition (np.exp, a - b, ...), rounded
nowhere; tolerances 1e-5 (fp32) / 1e-2 (bf16, fp16) / 1e-12 (fp64)."""
import numpy as np
import pytest

import helpers
import oracle

pytestmark = pytest.mark.gpu

DTYPES = ["fp32", "bf16", "fp16", "fp64"]
NP_UNARY = {"exp": np.exp, "log": np.log, "neg": np.negative, "sqrt": np.sqrt}
NP_BINARY = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}


def _draw(seed, shape, dtype, positive=False):
    g = helpers.rng(seed)
    v = g.standard_normal(shape) if not positive else g.uniform(0.5, 4.0, shape)
    return v.astype(np.float64) if dtype == "fp64" else oracle.round_to(v.astype(np.float32), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["exp", "log", "neg", "sqrt"])
@pytest.mark.parametrize("n", [1, 7, 4096, 100003, 1 << 20])
def test_unary(hk, cuda, dtype, op, n):
    import torch
    x = _draw(11 + n, (n,), dtype, positive=op in ("log", "sqrt"))
    tx = helpers.to_torch(x, dtype, cuda)
    ty = torch.empty_like(tx)
    hk.unary(op, tx, ty)
    torch.cuda.synchronize()
    helpers.assert_close(ty, NP_UNARY[op](x.astype(np.float64)), dtype, op)
    # in place, and from an address that is not 16-byte aligned
    if n > 8:
        tv = tx[1:]
        hk.unary(op, tv, tv)
        torch.cuda.synchronize()
        helpers.assert_close(tv, NP_UNARY[op](x[1:].astype(np.float64)), dtype, op + " in place")


def test_unary_special_values(hk, cuda):
    import torch
    x = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 88.0, -80.0, 1e-30], device=cuda)
    y = torch.empty_like(x)
    hk.unary("exp", x, y)
    torch.cuda.synchronize()
    assert torch.allclose(y, torch.exp(x), rtol=1e-6, atol=0, equal_nan=True)
    hk.unary("log", x, y)
    torch.cuda.synchronize()
    assert torch.allclose(y, torch.log(x), rtol=1e-6, atol=0, equal_nan=True)
    hk.unary("sqrt", x, y)
    torch.cuda.synchronize()
    assert torch.allclose(y, torch.sqrt(x), rtol=1e-6, atol=0, equal_nan=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op,first", [("add", False), ("mul", False), ("sub", True), ("div", True), ("sub", False),
                                      ("div", False)])
@pytest.mark.parametrize("n", [5, 8192, 100003])
def test_binary_const(hk, cuda, dtype, op, first, n):
    import torch
    x = _draw(21 + n, (n,), dtype, positive=True)
    c = 1.0 / 3.0
    # the constant enters rounded to the array's type (static_cast<spec_t>(value) in the reference)
    cr = c if dtype == "fp64" else float(oracle.round_to(np.array([c], np.float32), dtype)[0])
    xd = x.astype(np.float64)
    want = NP_BINARY[op](cr, xd) if first else NP_BINARY[op](xd, cr)
    tx = helpers.to_torch(x, dtype, cuda)
    ty = torch.empty_like(tx)
    hk.binary_const(op, tx, c, ty, scalar_first=first)
    torch.cuda.synchronize()
    helpers.assert_close(ty, want, dtype, op)
    if dtype == "bf16" and op == "mul" and n >= 8192:
        # one fp32 product, one rounding: bit-exact with the constant rounded to bf16 first (bf16(1/3) lies 2e-3
        # above 1/3), and visibly different from the product with the unrounded constant
        got = helpers.to_numpy(ty)
        assert np.array_equal(got, oracle.round_to(x.astype(np.float32) * np.float32(cr), "bf16"))
        assert (got != oracle.round_to(x.astype(np.float32) * np.float32(c), "bf16")).mean() > 0.2


BROADCASTS = [
    ((64, 4096), (64, 4096)),          # same shape
    ((64, 4096), (64, 1)),             # per-row value (logits - row maximum)
    ((64, 4096), (4096,)),             # per-column vector
    ((64, 1), (1, 4096)),              # outer combination
    ((64, 4096), ()),                  # single value
    ((3, 5, 7, 16), (5, 1, 16)),       # merges to nothing two-dimensional: generic kernel
    ((6, 10, 256), (6, 10, 1)),        # leading dims merge: [60, 256] op [60, 1]
    ((33, 1001), (33, 1)),             # odd row length: scalar path
    ((1,), (1,)),
    ((2, 3, 4, 5, 6, 2, 3, 2), (2, 1, 4, 1, 6, 1, 3, 1)),   # eight dims
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("shapes", BROADCASTS, ids=lambda s: "%sx%s" % s)
def test_binary_broadcast(hk, cuda, dtype, op, shapes):
    import torch
    sa, sb = shapes
    a = _draw(31, sa, dtype, positive=True)
    b = _draw(32, sb, dtype, positive=True)
    want = NP_BINARY[op](a.astype(np.float64), b.astype(np.float64))
    ta, tb = helpers.to_torch(a, dtype, cuda), helpers.to_torch(b, dtype, cuda)
    out = torch.empty(want.shape, dtype=ta.dtype, device=cuda)
    hk.binary(op, ta, tb, out)
    torch.cuda.synchronize()
    helpers.assert_close(out, want, dtype, op)
    # operands swapped (the broadcast one on the left)
    hk.binary(op, tb, ta, out)
    torch.cuda.synchronize()
    helpers.assert_close(out, NP_BINARY[op](b.astype(np.float64), a.astype(np.float64)), dtype, op + " swapped")


def test_binary_strided_operands_and_in_place(hk, cuda):
    import torch
    a = torch.randn(48, 512, device=cuda)
    b = torch.randn(512, 48, device=cuda)
    out = torch.empty(48, 512, device=cuda)
    hk.binary("add", a, b.t(), out)                       # transposed view: generic kernel
    torch.cuda.synchronize()
    assert torch.allclose(out, a + b.t(), rtol=1e-6, atol=1e-6)
    half = torch.empty(48, 256, device=cuda)
    hk.binary("mul", a[:, ::2], a[:, 1::2], half)         # column-strided views
    torch.cuda.synchronize()
    assert torch.allclose(half, a[:, ::2] * a[:, 1::2], rtol=1e-6, atol=1e-6)
    s = torch.rand(48, 1, device=cuda) + 0.5
    want = a / s
    hk.binary("div", a, s, a)                             # in place, as the loss op divides exp by its row sum
    torch.cuda.synchronize()
    assert torch.allclose(a, want, rtol=1e-6, atol=0)
    e = torch.empty(0, 16, device=cuda)
    hk.binary("add", e, e, e)                             # empty: nothing to do
    with pytest.raises(hk.HkError) as err:
        hk.binary("add", a > 0, a > 0, a > 0)             # bool is not an arithmetic type here
    assert err.value.code == -2
    with pytest.raises(hk.HkError) as err:
        hk.unary("exp", a.long(), a.long())               # exp / log / sqrt: floating types only
    assert err.value.code == -2


INT_TYPES = ["uint8", "int8", "int16", "int32", "int64"]


@pytest.mark.parametrize("tname", INT_TYPES)
def test_integer_types(hk, cuda, tname):
    """The reference dispatches add / sub / mul / div, their constant forms, negation and the broadcast kernels for
    the integer types too; integers are exact, so torch's own integer arithmetic is the expectation (wrapping in the
    type, division truncating toward zero)."""
    import torch
    td = getattr(torch, tname)
    g = torch.Generator(device="cuda").manual_seed(5)
    lo, hi = (0, 200) if tname == "uint8" else (-100, 100)
    a = torch.randint(lo, hi, (37, 129), generator=g, device=cuda).to(td)
    b = torch.randint(1, 9, (37, 129), generator=g, device=cuda).to(td)
    row = torch.randint(1, 9, (37, 1), generator=g, device=cuda).to(td)
    col = torch.randint(1, 9, (129,), generator=g, device=cuda).to(td)
    out = torch.empty_like(a)
    for name, fn in (("add", torch.add), ("sub", torch.sub), ("mul", torch.mul)):
        for other in (b, row, col):
            hk.binary(name, a, other, out)
            torch.cuda.synchronize()
            assert torch.equal(out, fn(a, other)), name
    hk.binary("div", a, b, out)
    torch.cuda.synchronize()
    assert torch.equal(out, torch.div(a, b, rounding_mode="trunc"))
    hk.binary_const("mul", a, 3, out)
    torch.cuda.synchronize()
    assert torch.equal(out, a * 3)
    hk.binary_const("sub", a, 7, out, scalar_first=True)
    torch.cuda.synchronize()
    assert torch.equal(out, 7 - a)
    hk.unary("neg", a, out)
    torch.cuda.synchronize()
    assert torch.equal(out, -a if tname != "uint8" else (256 - a.to(torch.int32)).remainder(256).to(td))
    wide = torch.empty(5, 37, 129, dtype=td, device=cuda)
    hk.broadcast(a, wide)
    torch.cuda.synchronize()
    assert torch.equal(wide, a.expand(5, 37, 129))
    hk.broadcast(row, out, scalar=2)
    torch.cuda.synchronize()
    assert torch.equal(out, (row * 2).expand(37, 129))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols", [1000, 4096, 50257])
def test_vocab_parallel_local_kernels(hk, cuda, dtype, cols):
    import torch
    rows, ignored = 77, -100
    start = 3 * cols
    g = helpers.rng(5 + cols)
    logits = _draw(41 + cols, (rows, cols), dtype)
    labels = g.integers(0, 8 * cols, rows).astype(np.int64)          # most labels lie in other shards
    labels[::5] = g.integers(start, start + cols, len(labels[::5]))  # every fifth in this one
    labels[3] = ignored; labels[10] = start; labels[11] = start + cols - 1; labels[12] = start + cols
    labels[13] = start - 1
    tl = helpers.to_torch(logits, dtype, cuda); tlab = torch.from_numpy(labels).to(cuda)
    picked = torch.full((rows,), 7.0, dtype=tl.dtype, device=cuda)
    lse = torch.full((rows,), 5.0, dtype=tl.dtype, device=cuda)
    hk.vocab_parallel_ce_gather(tl, tlab, start, start + cols, ignored, picked, lse)
    torch.cuda.synchronize()
    inside = (labels >= start) & (labels < start + cols) & (labels != ignored)
    want = np.where(inside, logits[np.arange(rows), np.clip(labels - start, 0, cols - 1)], 0.0)
    assert np.array_equal(helpers.to_numpy(picked).astype(np.float64), want.astype(np.float64))   # a gather: exact
    want_lse = np.where(labels == ignored, 0.0, 5.0)
    assert np.array_equal(helpers.to_numpy(lse).astype(np.float64), want_lse)

    sm = np.abs(_draw(43 + cols, (rows, cols), dtype)) / cols
    gl = _draw(44, (rows,), dtype)
    onehot = np.zeros((rows, cols)); onehot[np.flatnonzero(inside), (labels - start)[inside]] = 1.0
    want_grad = (sm.astype(np.float64) - onehot) * gl.astype(np.float64)[:, None]
    tsm, tgl = helpers.to_torch(sm, dtype, cuda), helpers.to_torch(gl, dtype, cuda)
    out = torch.empty_like(tsm)
    hk.vocab_parallel_ce_bwd(tsm, tlab, tgl, out, start)
    torch.cuda.synchronize()
    helpers.assert_close(out, want_grad, dtype, "gradient")
    hk.vocab_parallel_ce_bwd(tsm, tlab, tgl, tsm, start)   # in place
    torch.cuda.synchronize()
    assert torch.equal(tsm, out)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_vocab_parallel_loss_over_two_shards_equals_the_fused_loss(hk, cuda, dtype):
    """The loss op's sequence (VocabParallelCrossEntropyLoss.cc:51-108) on two column shards held by this one
    GPU, the three cross-device reductions replaced by max / sum over the two partial results: row maximum,
    logits - maximum, exp, row sum, divide (softmax kept), log, gather, subtract.  Its per-row loss and its
    gradient must equal the fused sparse cross-entropy of the whole matrix."""
    import torch
    rows, cols, ignored = 96, 4096, -100
    half = cols // 2
    g = helpers.rng(77)
    logits = _draw(51, (rows, cols), dtype) * 3
    labels = g.integers(0, cols, rows).astype(np.int64); labels[::9] = ignored
    full = helpers.to_torch(logits, dtype, cuda); tlab = torch.from_numpy(labels).to(cuda)
    loss_ref = oracle.sce_sparse_fwd(logits, labels, ignored)
    gl = np.where(labels == ignored, 0.0, 1.0 / rows)
    grad_ref = oracle.sce_sparse_bwd(logits, labels, gl.astype(np.float32), ignored)

    shards = [full[:, :half].contiguous(), full[:, half:].contiguous()]
    tdt = full.dtype
    col = lambda: torch.empty(rows, 1, dtype=tdt, device=cuda)
    part_max = []
    for x in shards:
        m = col()
        hk.reduce(x, m.view(rows), [1], "max")
        part_max.append(m)
    row_max = torch.maximum(part_max[0], part_max[1])                 # all-reduce(max)
    exps, part_sum = [], []
    for x in shards:
        v = torch.empty_like(x)
        hk.binary("sub", x, row_max, v)
        hk.unary("exp", v, v)
        s = col()
        hk.reduce(v, s.view(rows), [1], "sum")
        exps.append(v); part_sum.append(s)
    row_sum = part_sum[0] + part_sum[1]                               # all-reduce(sum)
    lse = col()
    hk.unary("log", row_sum, lse)
    picked_total = torch.zeros(rows, 1, dtype=torch.float32, device=cuda)
    grads = []
    tgl = helpers.to_torch(gl, dtype, cuda).view(rows, 1)
    for k, x in enumerate(shards):
        shifted = torch.empty_like(x)
        hk.binary("sub", x, row_max, shifted)
        picked = col()
        lse_k = lse.clone()
        hk.vocab_parallel_ce_gather(shifted, tlab, k * half, (k + 1) * half, ignored, picked.view(rows),
                                    lse_k.view(rows))
        picked_total += picked.float()                                # all-reduce(sum)
        hk.binary("div", exps[k], row_sum, exps[k])                   # softmax, in place
        out = torch.empty_like(x)
        hk.vocab_parallel_ce_bwd(exps[k], tlab, tgl.view(rows), out, k * half)
        grads.append(out)
        lse_final = lse_k
    loss = torch.empty(rows, 1, dtype=tdt, device=cuda)
    hk.binary("sub", lse_final, picked_total.to(tdt), loss)
    torch.cuda.synchronize()
    # In bf16 the unfused sequence rounds logits - maximum (up to ~25 in magnitude here) to 8 bits before the
    # exponential: an absolute error of up to 0.06 in the exponent, i.e. several percent in softmax.  That is the
    # arithmetic of the sequence itself (every step below is within 1e-2 of its own definition, tested above).
    helpers.assert_close(loss.view(rows), loss_ref, dtype, "loss", rtol=2e-2 if dtype == "bf16" else 1e-5)
    helpers.assert_close(torch.cat(grads, dim=1), grad_ref, dtype, "gradient",
                         rtol=1e-1 if dtype == "bf16" else 1e-5)


def test_division_by_a_per_row_value_is_correctly_rounded(hk, cuda):
    """The per-row divisor path forms one reciprocal per row and corrects each quotient twice; the result must
    be the correctly rounded fp32 quotient, bit for bit, over the whole exponent range, zeros, infinities, NaN
    and denormals included (torch's fp32 division is IEEE and serves as the reference)."""
    import torch
    rows, cols = 4096, 4096
    g = torch.Generator(device="cuda").manual_seed(1)
    mant = torch.rand(rows, cols, generator=g, device=cuda) + 1.0
    expo = torch.randint(-60, 60, (rows, cols), generator=g, device=cuda)
    a = torch.ldexp(mant, expo) * torch.where(torch.rand(rows, cols, generator=g, device=cuda) < 0.5, -1.0, 1.0)
    b = torch.ldexp(torch.rand(rows, 1, generator=g, device=cuda) + 1.0,
                    torch.randint(-126, 127, (rows, 1), generator=g, device=cuda))
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-45, -3e-39, 3e38, 1.0, 3.0],
                           device=cuda)
    a[:, :10] = special
    b[:10, 0] = special
    out = torch.empty_like(a)
    hk.binary("div", a, b, out)
    torch.cuda.synchronize()
    want = a / b
    same = (out.view(torch.int32) == want.view(torch.int32)) | (torch.isnan(out) & torch.isnan(want))
    assert bool(same.all()), "%d of %d quotients differ from the correctly rounded ones" % (int((~same).sum()), same.numel())


def test_bf16_division_rounds_like_the_exact_quotient(hk, cuda):
    """bf16 quotients are formed with the hardware reciprocal; every bf16 bit pattern as dividend against 4096
    divisors (random, plus zeros, infinities, NaN, denormals, extremes), full and per-row operand modes: bit
    for bit the bf16 rounding of the IEEE fp32 quotient."""
    import torch
    a = torch.arange(65536, device=cuda, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)   # all patterns
    g = torch.Generator(device="cuda").manual_seed(2)
    b = torch.randint(0, 65536, (4096,), generator=g, device=cuda, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    b[:8] = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-40, 3e38, 1.0], device=cuda).bfloat16()
    A = a.view(1, 65536).expand(4096, 65536).contiguous()
    out = torch.empty_like(A)
    for bb in (b.view(4096, 1), b.view(4096, 1).expand(4096, 65536).contiguous()):
        hk.binary("div", A, bb, out)
        torch.cuda.synchronize()
        want = (A.float() / bb.float()).bfloat16()
        same = (out.view(torch.int16) == want.view(torch.int16)) | (torch.isnan(out) & torch.isnan(want))
        assert bool(same.all()), "%d of %d bf16 quotients differ" % (int((~same).sum()), same.numel())


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16", "fp64"])
@pytest.mark.parametrize("rows,cols,nshards", [(96, 4096, 2), (33, 32000, 4), (50, 1000, 5), (7, 24, 3)])
def test_vocab_parallel_fused_form_equals_the_whole_row_loss(hk, cuda, dtype, rows, cols, nshards):
    """One read per shard (row maximum, sum of exponentials, picked logit), a per-row combination of the shards'
    statistics, and a backward that rebuilds softmax from logits and log-sum-exp: loss and gradient must equal
    the cross-entropy of the unsplit matrix; ignored rows give loss 0 and a zero gradient; the label gather is
    exact."""
    import torch
    ignored = -100
    g = helpers.rng(rows + cols)
    logits = _draw(61 + cols, (rows, cols), dtype) * 3
    if dtype != "fp64":
        logits = oracle.round_to(logits.astype(np.float32), dtype)
    labels = g.integers(0, cols, rows).astype(np.int64); labels[::6] = ignored
    loss_ref = oracle.sce_sparse_fwd(logits, labels, ignored) if dtype != "fp64" else None
    if dtype == "fp64":
        m = logits.max(axis=1, keepdims=True)
        lse64 = (np.log(np.exp(logits - m).sum(axis=1)) + m[:, 0])
        loss_ref = np.where(labels == ignored, 0.0, lse64 - logits[np.arange(rows), np.clip(labels, 0, cols - 1)])
    gl = _draw(62, (rows,), dtype)
    sm = np.exp(logits.astype(np.float64) - logits.astype(np.float64).max(axis=1, keepdims=True))
    sm /= sm.sum(axis=1, keepdims=True)
    onehot = np.zeros((rows, cols)); keep = labels != ignored
    onehot[np.flatnonzero(keep), labels[keep]] = 1.0
    grad_ref = np.where(keep[:, None], (sm - onehot) * gl.astype(np.float64)[:, None], 0.0)

    full = helpers.to_torch(logits, dtype, cuda); tlab = torch.from_numpy(labels).to(cuda)
    width = cols // nshards
    bounds = [(k * width, cols if k == nshards - 1 else (k + 1) * width) for k in range(nshards)]
    shards = [full[:, lo:hi].contiguous() for lo, hi in bounds]
    stats = torch.empty(nshards, 3, rows, dtype=torch.float32, device=cuda)
    for k, (lo, hi) in enumerate(bounds):
        hk.vocab_parallel_ce_stats(shards[k], tlab, stats[k], lo, ignored)
    torch.cuda.synchronize()
    # the gather is exact, and falls into exactly one shard per row
    picked = stats[:, 2, :].sum(dim=0).cpu().numpy().astype(np.float64)
    want_picked = np.where(keep, logits[np.arange(rows), np.clip(labels, 0, cols - 1)], 0.0).astype(np.float64)
    if dtype != "fp64":
        assert np.array_equal(picked, want_picked)
    loss = torch.empty(rows, dtype=full.dtype, device=cuda)
    lse = torch.empty(rows, dtype=torch.float32, device=cuda)
    hk.vocab_parallel_ce_combine(stats, tlab, ignored, loss, lse)     # stats as an all-gather would leave them
    tgl = helpers.to_torch(gl, dtype, cuda)
    grads = []
    for k, (lo, hi) in enumerate(bounds):
        out = torch.empty_like(shards[k])
        hk.vocab_parallel_ce_bwd_fused(shards[k], tlab, lse, tgl, out, lo, ignored)
        grads.append(out)
    torch.cuda.synchronize()
    tol = {"fp64": 1e-5}.get(dtype)      # statistics and log-sum-exp are fp32 whatever the logits' type
    helpers.assert_close(loss, loss_ref, dtype, "loss", rtol=tol)
    assert (helpers.to_numpy(loss)[~keep] == 0).all()
    got = torch.cat(grads, dim=1)
    helpers.assert_close(got, grad_ref, dtype, "gradient", rtol=tol)
    assert (helpers.to_numpy(got)[~keep] == 0).all()
    # in place on the logits, as a caller short of memory would run it
    hk.vocab_parallel_ce_bwd_fused(shards[0], tlab, lse, tgl, shards[0], bounds[0][0], ignored)
    torch.cuda.synchronize()
    assert torch.equal(shards[0], grads[0])


def test_vocab_parallel_stats_of_one_shard_match_their_definition(hk, cuda):
    import torch
    rows, cols, start = 40, 5120, 10240
    x = torch.randn(rows, cols, device=cuda) * 4
    x[3] = -float("inf")                                  # a shard with no finite logit
    x[4, :100] = float("inf")
    labels = torch.randint(start, start + cols, (rows,), device=cuda); labels[5] = start - 7; labels[6] = -100
    stats = torch.empty(3, rows, device=cuda)
    hk.vocab_parallel_ce_stats(x, labels, stats, start, -100)
    torch.cuda.synchronize()
    m = x.max(dim=1).values
    keep = torch.ones(rows, dtype=torch.bool, device=cuda); keep[6] = False
    assert torch.equal(stats[0][keep], m[keep]) and stats[0][6] == -float("inf")
    s = torch.exp(x - m[:, None]).sum(dim=1)
    fin = torch.isfinite(m) & keep
    assert torch.allclose(stats[1][fin], s[fin], rtol=1e-5)
    assert stats[1][3] == 0 and stats[1][6] == 0
    local = (labels - start).clamp(0, cols - 1)
    want = torch.where((labels >= start) & (labels < start + cols) & keep, x[torch.arange(rows), local], torch.zeros(()).to(x))
    assert torch.equal(stats[2], want)
